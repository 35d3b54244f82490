"""Python face of the HIP kernel library: one function per kernel, each checking on the host that
operand shapes, types and devices are what the kernel and its grid assume before anything is launched.

All work goes to torch's current stream.  There is no CPU path: a tensor that is not on the GPU, or a
missing library, raises.
"""
from __future__ import annotations

import ctypes
import sys
from typing import Optional

import torch

from . import build

F32, BF16 = 0, 1
_CODES = {1: "bad argument", 2: "unsupported size", 3: "launch failed"}

_c_int, _c_ll, _c_float, _c_ptr = ctypes.c_int, ctypes.c_longlong, ctypes.c_float, ctypes.c_void_p

_SIGNATURES = {
    "ms_embed": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "ms_rms_norm": [_c_ptr, _c_ptr, _c_int, _c_int, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int,
                    _c_int, _c_ptr],
    "ms_rms_norm_pair": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "ms_gemm_skinny_norm": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_int,
                            _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_qkv_rope_store": [_c_ptr, _c_ll, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_decode_advance": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
                          _c_int, _c_ptr],
    "ms_max_cache_groups": [],
    "ms_table_update": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ll, _c_ptr],
    "ms_zero_rows": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_int, _c_ptr],
    "ms_bias_add": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "ms_gemm_skinny": [_c_ptr, _c_ll, _c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int,
                       _c_ptr],
    "ms_gemm_stream": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int,
                       _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_gemm_panel": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int,
                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_gemm_panel_splitk_parts": [_c_int, _c_int, _c_int],
    "ms_gemm_panel_splitk": [_c_ptr, _c_ll, _c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int,
                             _c_ptr, _c_int, _c_ptr],
    "ms_gemm_tiled": [_c_ptr, _c_ll, _c_ptr, _c_ll, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_gemm_tiled_force": [_c_int],
    "ms_gemm_tiled_force_xcd_split": [_c_int],
    "ms_gemm_tiled_pays": [_c_int, _c_int, _c_int],
    "ms_gemm_tiled_plain_pays": [_c_int, _c_int, _c_int],
    "ms_gemm_tiled_qkv": [_c_ptr, _c_ll, _c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_rope_table": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
    "ms_gemm_tiled_qkv_pays": [_c_int, _c_int, _c_int, _c_int],
    "ms_read_probe_blocks": [],
    "ms_read_probe": [_c_ptr, _c_ll, _c_ptr, _c_ptr],
    "ms_residual_add": [_c_ptr, _c_ptr, _c_ll, _c_int, _c_ptr],
    "ms_silu_mul": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "ms_rope_store": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
                      _c_int, _c_int, _c_int, _c_ptr],
    "ms_gemm_generic": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ll, _c_ll, _c_ll, _c_int,
                        _c_int, _c_int, _c_ptr],
    "ms_paged_attention_generic": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                   _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ll, _c_float, _c_int, _c_int,
                                   _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ll, _c_float, _c_int, _c_ptr],
    "ms_attention_mfma_supported": [_c_int, _c_int],
    "ms_paged_attention_mfma": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll,
                                _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr,
                                _c_float, _c_ptr, _c_ptr, _c_ll, _c_float, _c_ptr],
    "ms_paged_attention_mfma_decode": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                       _c_ll, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                       _c_int, _c_int, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ll, _c_float, _c_ptr],
    "ms_argmax": [_c_ptr, _c_ll, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr],
    "ms_sample": [_c_ptr, _c_ll, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                  _c_ptr],
    "ms_sample_workspace_bytes": [_c_int],
    "ms_short_conv": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int,
                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_gated_delta": [_c_ptr, _c_ptr, _c_ptr, _c_ll, _c_ptr, _c_int, _c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                       _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_gated_head_norm": [_c_ptr, _c_ptr, _c_ptr, _c_ll, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_float,
                           _c_int, _c_ptr],
    "ms_gelu_tanh_glu": [_c_ptr, _c_ll, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_ptr],
    "ms_decay_recurrence": [_c_ptr, _c_ptr, _c_ptr, _c_ll, _c_ll, _c_ll, _c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_float,
                            _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr,
                            _c_int, _c_ptr],
    "ms_token_shift": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                       _c_int, _c_ptr],
    "ms_pair_sum": [_c_ptr, _c_ptr, _c_float, _c_float, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "ms_tanh": [_c_ptr, _c_ll, _c_int, _c_ptr],
    "ms_concat_rows": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_xielu": [_c_ptr, _c_ptr, _c_ptr, _c_ll, _c_int, _c_ptr],
    "ms_head_matmul": [_c_ptr, _c_ll, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_ll, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int,
                       _c_int, _c_int, _c_ptr],
    "ms_rms_norm_rows": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "ms_rotary_pairs": [_c_ptr, _c_ll, _c_ll, _c_ptr, _c_ll, _c_ll, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
                        _c_ptr],
    "ms_latent_kv_store": [_c_ptr, _c_ll, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                           _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_latent_attention_mfma": [_c_ptr, _c_ll, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                 _c_ptr, _c_ll, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ll, _c_float,
                                 _c_int, _c_ptr],
    "ms_latent_attention": [_c_ptr, _c_ll, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                            _c_ptr, _c_ll, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ll, _c_float, _c_int, _c_int,
                            _c_ptr],
    "ms_rms_norm_add": [_c_ptr, _c_ll, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_int, _c_int, _c_int,
                        _c_ptr],
    "ms_add_rows": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
    "ms_qk_norm_store": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_float, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
                         _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_ptr],
    "ms_selective_scan": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_ptr, _c_ptr,
                          _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_gelu": [_c_ptr, _c_ptr, _c_ll, _c_int, _c_ptr],
    "ms_moe_route": [_c_ptr, _c_ll, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr],
    "ms_layer_norm": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "ms_side_gate": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "ms_mingru_chunk": [],
    "ms_mingru_scan": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_ptr,
                       _c_int, _c_ptr],
    "ms_pairs_rotate_store": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                              _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_pool_store": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_pooled_attention": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr,
                            _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                            _c_int, _c_int, _c_int, _c_ptr],
    "ms_pooled_attention_mfma": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr,
                                 _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                 _c_int, _c_int, _c_ptr],
    "ms_clamped_glu": [_c_ptr, _c_ll, _c_ptr, _c_ll, _c_int, _c_int, _c_float, _c_float, _c_int, _c_ptr],
    "ms_scaled_swiglu": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_ptr],
    "ms_moe_tile_rows": [],
    "ms_moe_wide_tile_rows": [],
    "ms_gemm_tiled_grouped_rows": [],
    "ms_moe_align": [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr],
    "ms_grouped_gemm_mfma_ok": [_c_int, _c_ll, _c_ll, _c_int, _c_int, _c_int],
    "ms_grouped_gemm": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                        _c_int, _c_int, _c_int, _c_ptr],
    "ms_moe_combine": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll, _c_ptr, _c_int, _c_ptr, _c_ll, _c_ptr, _c_int, _c_int, _c_int,
                       _c_int, _c_int, _c_ptr],
}

_fn = {}


def _get(name):
    f = _fn.get(name)
    if f is None:
        lib = build.load()
        try:
            f = getattr(lib, name)
        except AttributeError as e:
            raise build.KernelLibraryError(
                f"{name} is not in {build.library_path()}; the library is older than its sources, build it again") from e
        f.argtypes = _SIGNATURES[name]
        f.restype = _c_int
        _fn[name] = f
    return f


class UnsupportedShape(RuntimeError):
    """A kernel has no variant for the sizes it was given (it launched nothing); another kernel may."""


def _call(name, *args):
    rc = _get(name)(*args)
    if rc == 2:
        raise UnsupportedShape(f"{name} refused its arguments: unsupported size (it has no variant for these sizes)")
    if rc != 0:
        raise RuntimeError(f"{name} refused its arguments: {_CODES.get(rc, rc)}")


_said = set()


def _say_once(key, message: str) -> None:
    """A notice on stderr, once per process and key: a slower kernel than one might expect is in use."""
    if key not in _said:
        _said.add(key)
        print(f"[llm_infrence_engine_amd] {message}", file=sys.stderr, flush=True)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current device's current stream as the handle the C entry points take.  Asked for at every launch:
    the accessors that build no Python object take 0.3 us against 8 us."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise TypeError(f"kernels take float32 or bfloat16, not {dtype}")


def _check(t: torch.Tensor, name: str, dtype=None, shape=None, contiguous=True):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} is on {t.device}; the kernels run on the GPU only (there is no CPU path)")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if contiguous and not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if shape is not None:
        have = t.shape
        ok = len(have) == len(shape)
        if ok:
            for s, a in zip(shape, have):     # a plain loop: this runs several times per kernel launch
                if s is not None and s != a:
                    ok = False
                    break
        if not ok:
            raise ValueError(f"{name} must have shape {list(shape)}, got {list(have)}")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


# ------------------------------------------------------------------------------------------------
def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[n] = float(table[ids[n]]) * scale.  ids int32 [N] (checked against the table by the caller), out float32 [N, H]."""
    _check(ids, "ids", torch.int32)
    _check(table, "table")
    V, H = table.shape
    _check(out, "out", torch.float32, (ids.numel(), H))
    _call("ms_embed", ids.data_ptr(), table.data_ptr(), out.data_ptr(), ids.numel(), H, float(scale), _code(table.dtype),
          _stream())
    return out


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
             delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
             write_back: bool = True) -> torch.Tensor:
    """out[r] = weight * normalised(x[rows[r]] (+ delta[rows[r]])).  x float32 [N, H] is the residual stream;
    with ``delta`` ([N, H], or partial sums [S, N, H] added in order) the sum is written back to x (unless
    ``write_back`` is False)."""
    _check(x, "x", torch.float32)
    N, H = x.shape
    _check(weight, "weight", torch.float32, (H,))
    n_rows = N
    if rows is not None:
        _check(rows, "rows", torch.int32)
        n_rows = rows.numel()
    _check(out, "out", None, (n_rows, H))
    dcode, n_partials = 0, 1
    if delta is not None:
        if delta.dim() == 3:
            n_partials = delta.shape[0]
            _check(delta, "delta", None, (n_partials, N, H))
        else:
            _check(delta, "delta", None, (N, H))
        dcode = _code(delta.dtype)
    _call("ms_rms_norm", x.data_ptr(), _ptr(delta), dcode, n_partials, N * H, weight.data_ptr(), _ptr(rows),
          out.data_ptr(), n_rows, H, float(eps), int(write_back), _code(out.dtype), _stream())
    return out


def rms_norm_pair(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, eps: float, out1: torch.Tensor, out2: torch.Tensor,
                  delta: Optional[torch.Tensor] = None):
    """out1 = w1 * normalised(x (+ delta)), out2 = w2 * normalised(x (+ delta)): two norms of the same rows of the float
    residual stream in one pass; with ``delta`` [N, H] the sum is written back to x."""
    _check(x, "x", torch.float32)
    N, H = x.shape
    _check(w1, "w1", torch.float32, (H,))
    _check(w2, "w2", torch.float32, (H,))
    _check(out1, "out1", None, (N, H))
    _check(out2, "out2", out1.dtype, (N, H))
    dcode = 0
    if delta is not None:
        _check(delta, "delta", None, (N, H))
        dcode = _code(delta.dtype)
    _call("ms_rms_norm_pair", x.data_ptr(), _ptr(delta), dcode, w1.data_ptr(), w2.data_ptr(), out1.data_ptr(),
          out2.data_ptr(), N, H, float(eps), _code(out1.dtype), _stream())
    return out1, out2


def bias_add(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x[n, :] += bias, in place."""
    _check(x, "x")
    _check(bias, "bias", torch.float32, (x.shape[-1],))
    _call("ms_bias_add", x.data_ptr(), bias.data_ptr(), x.numel() // x.shape[-1], x.shape[-1], _code(x.dtype), _stream())
    return x


MAX_CACHE_GROUPS = 8   # cache groups one call of ``decode_advance`` or ``table_update`` serves (the library's MS_MAX_GROUPS)


def max_cache_groups() -> int:
    """The same number, as the loaded library states it."""
    n = int(_get("ms_max_cache_groups")())
    if n != MAX_CACHE_GROUPS:
        raise build.KernelLibraryError(f"the library serves {n} cache groups, this module expects {MAX_CACHE_GROUPS}")
    return n


def _pointer_array(tensors):
    arr = (ctypes.c_void_p * max(1, len(tensors)))(*[t.data_ptr() for t in tensors])
    return arr, ctypes.cast(arr, ctypes.c_void_p)


def decode_advance(prev_tokens: torch.Tensor, token_ids: torch.Tensor, positions: torch.Tensor,
                   context_lens: torch.Tensor, n_live: torch.Tensor, table_rows: Optional[torch.Tensor], tables, slots,
                   page_size: int, draw_index: Optional[torch.Tensor] = None, strides=None) -> None:
    """Between two decode steps queued back to back: rows below ``n_live[0]`` move one position on, take
    ``prev_tokens`` as their input, count ``draw_index`` up by one and get their new slots from ``tables`` (one
    [table rows, width] per cache group; row r of the batch has the table row ``table_rows[r]``, or r without it).
    ``strides``: per group the tokens an entry stands for (1, the default: an entry per token; s > 1: the group stores with
    the last token of a block of s, other tokens get the slot -1)."""
    R = token_ids.numel()
    for t, name in ((prev_tokens, "prev_tokens"), (token_ids, "token_ids"), (positions, "positions"),
                    (context_lens, "context_lens")):
        _check(t, name, torch.int32, (R,))
    _check(n_live, "n_live", torch.int32, (1,))
    if len(tables) != len(slots) or len(tables) > max_cache_groups():
        raise ValueError(f"at most {max_cache_groups()} cache groups, one table and one slot mapping each")
    width = tables[0].shape[1] if tables else 1
    if table_rows is not None:
        _check(table_rows, "table_rows", torch.int32, (R,))
    if draw_index is not None:
        _check(draw_index, "draw_index", torch.int32, (R,))
    for t, sl in zip(tables, slots):
        _check(t, "table", torch.int32, (None if table_rows is not None else R, width))
        _check(sl, "slots", torch.int32, (R,))
    keep_t, tp = _pointer_array(tables)
    keep_s, sp = _pointer_array(slots)
    st = (ctypes.c_int * max(1, len(tables)))(*[int(v) for v in (strides or [1] * len(tables))])
    _call("ms_decode_advance", prev_tokens.data_ptr(), token_ids.data_ptr(), positions.data_ptr(),
          context_lens.data_ptr(), n_live.data_ptr(), _ptr(table_rows), _ptr(draw_index), tp, sp,
          ctypes.cast(st, ctypes.c_void_p), len(tables), width,
          page_size, R, _stream())


def table_update(tables, index, value, counts: torch.Tensor, max_updates: int) -> None:
    """tables[g].view(-1)[index[g][i]] = value[g][i] for i < counts[g]: the entries of the device's block tables
    that changed since the last step.  ``index`` / ``value``: per group int32 [max_updates]; ``counts`` int32
    [groups] on the device.  An index appears at most once per group."""
    G = len(tables)
    if not (G == len(index) == len(value)) or G > max_cache_groups():
        raise ValueError(f"one index and one value array per table, at most {max_cache_groups()} tables")
    if G == 0 or max_updates <= 0:
        return
    _check(counts, "counts", torch.int32, (G,))
    elems = tables[0].numel()
    for t, ix, v in zip(tables, index, value):
        _check(t, "table", torch.int32)
        if t.numel() != elems:
            raise ValueError("the block tables of all groups have one shape")
        _check(ix, "index", torch.int32, (max_updates,))
        _check(v, "value", torch.int32, (max_updates,))
    keep_t, tp = _pointer_array(tables)
    keep_i, ip = _pointer_array(index)
    keep_v, vp = _pointer_array(value)
    _call("ms_table_update", tp, ip, vp, counts.data_ptr(), G, max_updates, elems, _stream())


def zero_rows(t: torch.Tensor, rows: torch.Tensor, count: Optional[torch.Tensor] = None) -> torch.Tensor:
    """t[rows[i]] = 0 for every i (for i < count[0] with ``count``, a device int): rows of a tensor whose first
    dimension is indexed by ``rows``."""
    _check(t, "t")
    _check(rows, "rows", torch.int32)
    if count is not None:
        _check(count, "count", torch.int32, (1,))
    row_bytes = (t.numel() // max(1, t.shape[0])) * t.element_size()
    if row_bytes % 4:
        raise ValueError("rows must be a multiple of 4 bytes long")
    _call("ms_zero_rows", t.data_ptr(), row_bytes, rows.data_ptr(), _ptr(count), rows.numel(), _stream())
    return t


def read_probe(t: torch.Tensor) -> torch.Tensor:
    """Stream ``t`` once from memory with a kernel that does nothing else (for bandwidth measurements).
    Returns the exclusive-or of its 32-bit words per block."""
    _check(t, "t")
    nbytes = t.numel() * t.element_size()
    if nbytes % 16:
        raise ValueError("the probe reads multiples of 16 bytes")
    sink = torch.zeros(_get("ms_read_probe_blocks")(), dtype=torch.int32, device=t.device)
    _call("ms_read_probe", t.data_ptr(), nbytes, sink.data_ptr(), _stream())
    return sink


def residual_add(x: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _check(x, "x", torch.float32)
    _check(delta, "delta", None, tuple(x.shape))
    _call("ms_residual_add", x.data_ptr(), delta.data_ptr(), x.numel(), _code(delta.dtype), _stream())
    return x


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[n, i] = silu(gate_up[n, 2i]) * gate_up[n, 2i + 1]: gate and up columns interleaved."""
    _check(gate_up, "gate_up")
    N, two_i = gate_up.shape
    if two_i % 2:
        raise ValueError("gate_up must have an even number of columns")
    _check(out, "out", gate_up.dtype, (N, two_i // 2))
    _call("ms_silu_mul", gate_up.data_ptr(), out.data_ptr(), N, two_i // 2, _code(out.dtype), _stream())
    return out


def _v_shape(k_pages: torch.Tensor, v_transposed: bool, value_dim: Optional[int] = None):
    P, nkv, page_size, d = k_pages.shape
    d = d if value_dim is None else value_dim
    return (P, nkv, d, page_size) if v_transposed else (P, nkv, page_size, d)


def rope_store(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, rot_dim: int = 0,
               positions: Optional[torch.Tensor] = None, inv_freq: Optional[torch.Tensor] = None,
               slot_mapping: Optional[torch.Tensor] = None, k_pages: Optional[torch.Tensor] = None,
               v_pages: Optional[torch.Tensor] = None, v_transposed: bool = False,
               bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Add ``bias`` (if given), rotate q and k of ``qkv`` [N, (nh + 2 nkv) d] in place and store k, v into pages
    [pages, nkv, page_size, d] at ``slot_mapping`` (page * page_size + offset); with ``v_transposed`` the
    value pages are [pages, nkv, d, page_size]."""
    _check(qkv, "qkv", None, (None, (num_heads + 2 * num_kv_heads) * head_dim))
    N = qkv.shape[0]
    page_size = 0
    if rot_dim:
        if rot_dim % 2 or rot_dim > head_dim:
            raise ValueError(f"rot_dim {rot_dim} must be even and at most head_dim {head_dim}")
        _check(positions, "positions", torch.int32, (N,))
        _check(inv_freq, "inv_freq", torch.float32, (rot_dim // 2,))
    if k_pages is not None:
        _check(k_pages, "k_pages", qkv.dtype, (None, num_kv_heads, None, head_dim))
        page_size = k_pages.shape[2]
        _check(v_pages, "v_pages", qkv.dtype, _v_shape(k_pages, v_transposed))
        _check(slot_mapping, "slot_mapping", torch.int32, (N,))
    if bias is not None:
        _check(bias, "bias", torch.float32, (qkv.shape[1],))
    _call("ms_rope_store", qkv.data_ptr(), _ptr(bias), _ptr(positions), _ptr(inv_freq), _ptr(slot_mapping), _ptr(k_pages),
          _ptr(v_pages), N, num_heads, num_kv_heads, head_dim, rot_dim, page_size, int(v_transposed),
          _code(qkv.dtype), _stream())
    return qkv


def gemm_generic(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 accumulate: bool = False) -> torch.Tensor:
    """out (+)= a @ w.T (+ bias), float accumulation on the vector ALUs.  a [M, K] and out [M, N] may be row
    slices of wider matrices (unit stride in the last dimension)."""
    for t, name in ((a, "a"), (w, "w"), (out, "out")):
        _check(t, name, contiguous=False)
        if t.dim() != 2 or t.stride(1) != 1:
            raise ValueError(f"{name} must be a matrix with unit stride along its rows")
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or tuple(out.shape) != (M, N):
        raise ValueError(f"shapes do not fit: a {list(a.shape)}, w {list(w.shape)}, out {list(out.shape)}")
    if a.dtype != w.dtype:
        raise TypeError(f"a is {a.dtype} but w is {w.dtype}")
    if bias is not None:
        _check(bias, "bias", torch.float32, (N,))
    _call("ms_gemm_generic", a.data_ptr(), w.data_ptr(), _ptr(bias), out.data_ptr(), M, N, K,
          a.stride(0) if M > 1 else K, w.stride(0) if N > 1 else K, out.stride(0) if M > 1 else N,
          _code(a.dtype), _code(out.dtype), int(accumulate), _stream())
    return out


SKINNY_MAX_ROWS = 64
EPI_STORE, EPI_SWIGLU, EPI_RESIDUAL = 0, 1, 3
EPI_GEGLU = 4      # as EPI_SWIGLU with the tanh form of the gelu (the tiled product alone has it)


def skinny_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the few-rows matrix-core kernel takes this product."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[0] <= SKINNY_MAX_ROWS
            and a.shape[1] % 8 == 0 and a.stride(1) == 1 and w.is_contiguous()
            and (a.shape[0] == 1 or a.stride(0) % 8 == 0) and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, epilogue: int = EPI_STORE,
                out_dtype: torch.dtype = torch.bfloat16, residual: Optional[torch.Tensor] = None,
                split_columns: bool = True) -> torch.Tensor:
    """a [M <= 64, K] @ w [N, K].T on the matrix cores, bfloat16 in.  Epilogues: EPI_STORE -> [M, N] (+ bias);
    EPI_SWIGLU -> [M, N / 2] = silu(even rows' products) * odd rows' products; EPI_RESIDUAL -> ``residual``
    (float [M, N]) += product + bias, in place."""
    _check(a, "a", torch.bfloat16, contiguous=False)
    _check(w, "w", torch.bfloat16)
    if a.dim() != 2 or w.dim() != 2 or a.shape[1] != w.shape[1]:
        raise ValueError(f"shapes do not fit: a {list(a.shape)}, w {list(w.shape)}")
    if not skinny_ok(a, w):
        raise ValueError(f"the few-rows kernel takes at most {SKINNY_MAX_ROWS} rows of bfloat16 with K a multiple of 8 "
                         f"and 16-byte aligned rows; got a {list(a.shape)} strides {a.stride()}")
    M, K = a.shape
    N = w.shape[0]
    if bias is not None:
        _check(bias, "bias", torch.float32, (N,))
    if epilogue == EPI_STORE:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
        ldo = N
    elif epilogue == EPI_SWIGLU:
        if N % 2 or bias is not None:
            raise ValueError("the gated epilogue needs an even number of weight rows and no bias")
        out, ldo, out_dtype = torch.empty((M, N // 2), dtype=torch.bfloat16, device=a.device), N // 2, torch.bfloat16
    elif epilogue == EPI_RESIDUAL:
        _check(residual, "residual", torch.float32, (M, N))
        out, ldo, out_dtype = residual, N, torch.float32
    else:
        raise ValueError(f"unknown epilogue {epilogue}")
    lda = a.stride(0) if M > 1 else K
    if epilogue != EPI_SWIGLU and split_columns:
        # long rows against few of them (a down projection): the columns are split over blocks too, and the
        # partial sums are added up in a fixed order by a second kernel
        parts = _get("ms_gemm_panel_splitk_parts")(M, N, K)
        if parts > 1:
            partial = torch.empty((parts, M, N), dtype=torch.float32, device=a.device)
            _call("ms_gemm_panel_splitk", a.data_ptr(), lda, w.data_ptr(), K, _ptr(bias), out.data_ptr(), ldo, M, N, K,
                  epilogue, _code(out_dtype), partial.data_ptr(), parts, _stream())
            return out
    _call("ms_gemm_skinny", a.data_ptr(), lda, w.data_ptr(), K, _ptr(bias), out.data_ptr(), ldo,
          M, N, K, epilogue, _code(out_dtype), _stream())
    return out


def gemm_tiled_pays(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_tiled(a, w, EPI_SWIGLU)`` takes these sizes and is the faster way to the gated product."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and a.is_contiguous()
            and w.is_contiguous() and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and bool(_get("ms_gemm_tiled_pays")(a.shape[0], w.shape[0], a.shape[1])))


def gemm_tiled_plain_pays(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_tiled(a, w)`` is the better way to a plain product than the library's (short portions of a
    narrow model, where the host's time to enqueue a launch is what counts)."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and a.is_contiguous()
            and w.is_contiguous() and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and bool(_get("ms_gemm_tiled_plain_pays")(a.shape[0], w.shape[0], a.shape[1])))


def gemm_tiled(a: torch.Tensor, w: torch.Tensor, epilogue: int = EPI_STORE) -> torch.Tensor:
    """a [M, K] @ w [N, K].T for many rows on the matrix cores, bfloat16 in and out: EPI_STORE -> [M, N];
    EPI_SWIGLU over interleaved rows of w (2j: gate j, 2j + 1: up j) -> [M, N / 2], the product itself never
    written; EPI_GEGLU: the same with gelu_tanh(gate) for silu(gate).  K a multiple of 64 (else ``UnsupportedShape``)."""
    _check(a, "a", torch.bfloat16)
    _check(w, "w", torch.bfloat16, (None, a.shape[1]))
    if epilogue not in (EPI_STORE, EPI_SWIGLU, EPI_GEGLU):
        raise ValueError("the tiled product stores its result or the gated activation of it")
    M, K = a.shape
    N = w.shape[0]
    out = torch.empty((M, N // 2 if epilogue in (EPI_SWIGLU, EPI_GEGLU) else N), dtype=torch.bfloat16, device=a.device)
    _call("ms_gemm_tiled", a.data_ptr(), K, w.data_ptr(), K, out.data_ptr(), out.shape[1], M, N, K, epilogue, _stream())
    return out


def gemm_tiled_qkv_pays(a, w: torch.Tensor, head_dim: int, rot_dim: int, k_pages: torch.Tensor) -> bool:
    """Whether ``gemm_tiled_qkv`` takes these operands (bfloat16 rows, heads of 64 or 128 rotated whole) and is the
    faster way from a portion's normed rows to q and the cache."""
    return (isinstance(a, torch.Tensor) and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2
            and a.is_contiguous() and w.is_contiguous() and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and rot_dim == head_dim and k_pages.dtype == torch.bfloat16
            and bool(_get("ms_gemm_tiled_qkv_pays")(a.shape[0], w.shape[0], a.shape[1], head_dim)))


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """float [N, half, 2]: (cos, sin) of float(positions[n]) * inv_freq[j], for ``gemm_tiled_qkv``."""
    _check(positions, "positions", torch.int32)
    _check(inv_freq, "inv_freq", torch.float32)
    n, half = positions.numel(), inv_freq.numel()
    table = torch.empty((n, half, 2), dtype=torch.float32, device=positions.device)
    _call("ms_rope_table", positions.data_ptr(), inv_freq.data_ptr(), table.data_ptr(), n, half, _stream())
    return table


def gemm_tiled_qkv(a: torch.Tensor, w_qkv: torch.Tensor, bias: Optional[torch.Tensor], nh: int, nkv: int, d: int,
                   table: torch.Tensor, slot_mapping: torch.Tensor, k_pages: torch.Tensor,
                   v_pages: torch.Tensor, v_transposed: bool = False) -> torch.Tensor:
    """a [M, K] @ w_qkv [(nh + 2 nkv) d, K].T (+ bias) on the matrix cores with the rotation of q and k and the
    store of k and v into the pages as the product's epilogue; returns q [M, nh d].  ``table`` is
    ``rope_table(positions, inv_freq)`` with d / 2 frequencies (whole heads are rotated); pages as in
    ``rope_store``."""
    _check(a, "a", torch.bfloat16)
    M, K = a.shape
    _check(w_qkv, "w_qkv", torch.bfloat16, ((nh + 2 * nkv) * d, K))
    _check(table, "table", torch.float32, (M, d // 2, 2))
    _check(slot_mapping, "slot_mapping", torch.int32, (M,))
    if bias is not None:
        _check(bias, "bias", torch.float32, ((nh + 2 * nkv) * d,))
    _check(k_pages, "k_pages", torch.bfloat16, (None, nkv, None, d))
    page_size = k_pages.shape[2]
    _check(v_pages, "v_pages", torch.bfloat16, _v_shape(k_pages, v_transposed))
    q = torch.empty((M, nh * d), dtype=torch.bfloat16, device=a.device)
    _call("ms_gemm_tiled_qkv", a.data_ptr(), K, w_qkv.data_ptr(), K, _ptr(bias), table.data_ptr(),
          slot_mapping.data_ptr(), q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), M, K, nh,
          nkv, d, page_size, int(bool(v_transposed)), _stream())
    return q


def skinny_norm_ok(x: torch.Tensor, w: torch.Tensor, n_rows: int) -> bool:
    """Whether the few-rows kernel with the RMS norm folded in takes float rows of ``x`` against ``w``."""
    return (x.dtype == torch.float32 and w.dtype == torch.bfloat16 and n_rows <= SKINNY_MAX_ROWS and x.dim() == 2
            and x.shape[1] % 8 == 0 and x.is_contiguous() and w.is_contiguous() and x.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def gemm_skinny_norm(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, w: torch.Tensor,
                     bias: Optional[torch.Tensor] = None, epilogue: int = EPI_STORE,
                     out_dtype: torch.dtype = torch.bfloat16, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """rms_norm(x[rows]) @ w.T with the norm folded into the product: x float32 [N, K] is the residual stream,
    ``norm_weight`` float32 [K].  Epilogues EPI_STORE (+ bias) and EPI_SWIGLU as in ``gemm_skinny``."""
    _check(x, "x", torch.float32)
    _check(w, "w", torch.bfloat16)
    N_rows, K = x.shape
    M = N_rows
    if rows is not None:
        _check(rows, "rows", torch.int32)
        M = rows.numel()
    if w.shape[1] != K:
        raise ValueError(f"shapes do not fit: x {list(x.shape)}, w {list(w.shape)}")
    if not skinny_norm_ok(x, w, M):
        raise ValueError(f"the few-rows kernel takes at most {SKINNY_MAX_ROWS} float rows with K a multiple of 8")
    _check(norm_weight, "norm_weight", torch.float32, (K,))
    N = w.shape[0]
    if bias is not None:
        _check(bias, "bias", torch.float32, (N,))
    if epilogue == EPI_STORE:
        out, ldo = torch.empty((M, N), dtype=out_dtype, device=x.device), N
    elif epilogue == EPI_SWIGLU:
        if N % 2 or bias is not None:
            raise ValueError("the gated epilogue needs an even number of weight rows and no bias")
        out, ldo, out_dtype = torch.empty((M, N // 2), dtype=torch.bfloat16, device=x.device), N // 2, torch.bfloat16
    else:
        raise ValueError(f"epilogue {epilogue} is not available with the folded norm")
    _call("ms_gemm_skinny_norm", x.data_ptr(), K, _ptr(rows), norm_weight.data_ptr(), float(eps), w.data_ptr(), K,
          _ptr(bias), out.data_ptr(), ldo, M, N, K, epilogue, _code(out_dtype), _stream())
    return out


STREAM_MAX_ROWS = 16


def _gemm_by_name(entry: str, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], epilogue: int,
                  out_dtype: torch.dtype, residual: Optional[torch.Tensor], norm_weight: Optional[torch.Tensor],
                  eps: float, rows: Optional[torch.Tensor], any_shape: bool) -> torch.Tensor:
    norm = norm_weight is not None
    _check(a, "a", torch.float32 if norm else torch.bfloat16, contiguous=False)
    _check(w, "w", torch.bfloat16)
    if a.dim() != 2 or a.stride(1) != 1 or w.shape[1] != a.shape[1]:
        raise ValueError(f"shapes do not fit: a {list(a.shape)} (stride {a.stride()}), w {list(w.shape)}")
    K, N = a.shape[1], w.shape[0]
    M = a.shape[0]
    if rows is not None:
        _check(rows, "rows", torch.int32)
        M = rows.numel()
    if norm:
        _check(norm_weight, "norm_weight", torch.float32, (K,))
    if bias is not None:
        _check(bias, "bias", torch.float32, (N,))
    if epilogue == EPI_STORE:
        out, ldo = torch.empty((M, N), dtype=out_dtype, device=a.device), N
    elif epilogue == EPI_SWIGLU:
        out, ldo, out_dtype = torch.empty((M, N // 2), dtype=torch.bfloat16, device=a.device), N // 2, torch.bfloat16
    elif epilogue == EPI_RESIDUAL:
        _check(residual, "residual", torch.float32, (M, N))
        out, ldo, out_dtype = residual, N, torch.float32
    else:
        raise ValueError(f"unknown epilogue {epilogue}")
    _call(entry, a.data_ptr(), a.stride(0) if a.shape[0] > 1 else K, _ptr(rows), _ptr(norm_weight), float(eps),
          w.data_ptr(), K, _ptr(bias), out.data_ptr(), ldo, M, N, K, epilogue, _code(out_dtype), int(norm),
          int(any_shape), _stream())
    return out


def gemm_stream(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, epilogue: int = EPI_STORE,
                out_dtype: torch.dtype = torch.bfloat16, residual: Optional[torch.Tensor] = None,
                norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                rows: Optional[torch.Tensor] = None, any_shape: bool = True) -> torch.Tensor:
    """The streaming kernel for up to 16 rows, called by name (``gemm_skinny`` and ``gemm_skinny_norm`` go to it by
    themselves for the shapes it is faster on): ``a`` bfloat16 [M, K], or with ``norm_weight`` the float32
    residual stream whose RMS norm is folded in.  With ``any_shape`` every shape it can compute is taken;
    a shape it cannot raises."""
    return _gemm_by_name("ms_gemm_stream", a, w, bias, epilogue, out_dtype, residual, norm_weight, eps, rows, any_shape)


PANEL_MAX_ROWS = 64


def gemm_panel(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, epilogue: int = EPI_STORE,
               out_dtype: torch.dtype = torch.bfloat16, residual: Optional[torch.Tensor] = None,
               norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
               rows: Optional[torch.Tensor] = None, any_shape: bool = True) -> torch.Tensor:
    """The kernel that keeps up to 64 rows of activations whole in LDS, called by name (``gemm_skinny`` and
    ``gemm_skinny_norm`` go to it by themselves for more than 16 rows against a matrix of many rows).  Arguments
    as for ``gemm_stream``; a shape it cannot compute (rows that do not fit LDS) raises."""
    return _gemm_by_name("ms_gemm_panel", a, w, bias, epilogue, out_dtype, residual, norm_weight, eps, rows, any_shape)


def qkv_rope_store_ok(x: torch.Tensor, w: torch.Tensor, head_dim: int, rot_dim: int) -> bool:
    """Whether norm + projection + rotary + cache store can run as one kernel for these rows."""
    return skinny_norm_ok(x, w, x.shape[0]) and head_dim % 32 == 0 and rot_dim == head_dim


_cus = {}


def compute_units(device) -> int:
    """Compute units of the device (256 on an MI355X)."""
    key = torch.device(device).index or 0
    if key not in _cus:
        _cus[key] = torch.cuda.get_device_properties(key).multi_processor_count
    return _cus[key]


def qkv_rope_store_pays(x: torch.Tensor, w_qkv: torch.Tensor) -> bool:
    """Whether the one kernel is the faster way.  Each of its blocks (32 rows of the weight by 16 tokens) reads the
    float residual stream of its tokens again; as long as every block has a CU of its own that is cheaper than a
    kernel boundary, beyond that the norm, the product that holds the activations in LDS and the rotation win as
    kernels of their own (measured, 64 tokens: width 3,584 45 us fused against 29 + 6; width 5,120 86 against
    37 + 9; width 896 7 against 9 + 4)."""
    return (w_qkv.shape[0] // 32) * ((x.shape[0] + 15) // 16) <= compute_units(x.device)


def fold_norm_pays(n_rows: int, width: int) -> bool:
    """Whether a product should read the float residual stream and normalise it itself, rather than read bfloat16
    rows that a norm kernel of its own (3 to 4 us) has left.  Every block reads all rows of its tokens, so with
    many long rows the halved read is worth the launch (measured for the gated product: 64 rows of 3,584 82 against
    72 us, 32 rows of 5,120 129 against 120; 64 rows of 896 15.1 either way; 16 rows: folding wins at every width)."""
    return n_rows <= 16 or n_rows * width < 72 * 1024


def qkv_rope_store(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, w_qkv: torch.Tensor,
                   bias: Optional[torch.Tensor], num_heads: int, num_kv_heads: int, head_dim: int,
                   positions: torch.Tensor, inv_freq: torch.Tensor, slot_mapping: torch.Tensor,
                   k_pages: torch.Tensor, v_pages: torch.Tensor, v_transposed: bool) -> torch.Tensor:
    """rms_norm(x) @ w_qkv.T + bias, q and k rotated (whole head, half-split pairs), k and v stored into the
    pages at ``slot_mapping``; returns q bfloat16 [M, nh * d].  x float32 [M <= 64, K]."""
    _check(x, "x", torch.float32)
    M, K = x.shape
    _check(w_qkv, "w_qkv", torch.bfloat16, ((num_heads + 2 * num_kv_heads) * head_dim, K))
    if not qkv_rope_store_ok(x, w_qkv, head_dim, head_dim):
        raise ValueError("the fused projection takes at most 64 float rows, K a multiple of 8 and head sizes in steps of 32")
    _check(norm_weight, "norm_weight", torch.float32, (K,))
    if bias is not None:
        _check(bias, "bias", torch.float32, (w_qkv.shape[0],))
    _check(positions, "positions", torch.int32, (M,))
    _check(inv_freq, "inv_freq", torch.float32, (head_dim // 2,))
    _check(slot_mapping, "slot_mapping", torch.int32, (M,))
    _check(k_pages, "k_pages", torch.bfloat16, (None, num_kv_heads, None, head_dim))
    _check(v_pages, "v_pages", torch.bfloat16, _v_shape(k_pages, v_transposed))
    q = torch.empty((M, num_heads * head_dim), dtype=torch.bfloat16, device=x.device)
    _call("ms_qkv_rope_store", x.data_ptr(), K, norm_weight.data_ptr(), float(eps), w_qkv.data_ptr(), _ptr(bias),
          positions.data_ptr(), inv_freq.data_ptr(), slot_mapping.data_ptr(), q.data_ptr(), k_pages.data_ptr(),
          v_pages.data_ptr(), M, K, num_heads, num_kv_heads, head_dim, k_pages.shape[2], int(v_transposed), _stream())
    return q


def paged_attention_generic(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                            token_req: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, num_heads: int,
                            scale: float, window: Optional[int] = None, v_transposed: bool = False,
                            table_rows: Optional[torch.Tensor] = None,
                            n_live_tokens: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None,
                            softcap: float = 0.0, slopes: Optional[torch.Tensor] = None,
                            gate: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
    """out[n, h] = softmax(scale * q[n, h] . K[keys visible to n]) V, keys read in place from pages.

    q: [N, >= nh * d] (a row slice of the fused projection is fine), out [N, nh * d],
    pages [P, nkv, page_size, d] (values [P, nkv, d, page_size] with ``v_transposed``), block_table int32
    [rows, max_pages], token_req / positions int32 [N].
    Token n sees keys 0..positions[n] of request token_req[n] (the last ``window`` of them if given), whose
    pages are row ``table_rows[token_req[n]]`` of the table (row token_req[n] without ``table_rows``).  With
    ``n_live_tokens`` (a device int) tokens from that index on are left alone.  Values may have another size than
    keys (the value pages say which; out is then [N, nh * that size]).  ``sink`` float [nh]: exp(sink[h]) joins the
    denominator of head h's softmax.  ``softcap`` > 0: a scaled score s becomes softcap * tanh(s / softcap).  ``slopes``
    float [nh]: slopes[h] * (positions[n] - key's position) is taken off the score (after the cap).  ``gate`` [N, nh] (rows
    may be slices): head h's result is multiplied by sigmoid(gate[n, h]); ``out_scale`` multiplies every result."""
    _check(k_pages, "k_pages")
    P, nkv, page_size, d = k_pages.shape
    _check(v_pages, "v_pages", k_pages.dtype, (P, nkv, None, None))
    dv = v_pages.shape[2] if v_transposed else v_pages.shape[3]
    _check(v_pages, "v_pages", k_pages.dtype, _v_shape(k_pages, v_transposed, dv))
    _check(q, "q", k_pages.dtype, contiguous=False)
    N = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < num_heads * d:
        raise ValueError(f"q must be [N, >= {num_heads * d}] with unit stride along rows, got {list(q.shape)}")
    _check(out, "out", k_pages.dtype, (N, num_heads * dv))
    if sink is not None:
        _check(sink, "sink", torch.float32, (num_heads,))
    _check(block_table, "block_table", torch.int32)
    if block_table.dim() != 2:
        raise ValueError("block_table must be [requests, pages]")
    _check(token_req, "token_req", torch.int32, (N,))
    _check(positions, "positions", torch.int32, (N,))
    if table_rows is not None:
        _check(table_rows, "table_rows", torch.int32)
    if n_live_tokens is not None:
        _check(n_live_tokens, "n_live_tokens", torch.int32, (1,))
    if num_heads % nkv:
        raise ValueError(f"{num_heads} query heads cannot share {nkv} key/value heads")
    if slopes is not None:
        _check(slopes, "slopes", torch.float32, (num_heads,))
    gate_stride = _rows2d(gate, "gate", q.dtype, num_heads) if gate is not None else 0
    if gate is not None and gate.shape[0] != N:
        raise ValueError("gate must have a row per token")
    _call("ms_paged_attention_generic", q.data_ptr(), q.stride(0) if N > 1 else q.shape[1], k_pages.data_ptr(),
          v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], _ptr(table_rows), _ptr(n_live_tokens),
          token_req.data_ptr(), positions.data_ptr(),
          out.data_ptr(), num_heads * dv, N, num_heads, nkv, d, dv, page_size, P, float(scale), int(window or 0),
          int(v_transposed), _ptr(sink), float(softcap or 0.0), _ptr(slopes), _ptr(gate), gate_stride, float(out_scale),
          _code(q.dtype), _stream())
    return out


def attention_mfma_supported(head_dim: int, page_size: int) -> bool:
    return bool(_get("ms_attention_mfma_supported")(head_dim, page_size))


SPLIT_BLOCKS = 512         # blocks a split decode step's attention aims to put on the chip (two to a CU)
MAX_SPLITS = 16
MIN_BLOCKS_PER_SPLIT = 8   # of 32 keys
LONG_CONTEXT = 1024        # beyond this a decode batch also splits its keys over blocks
SPLIT_UP_TO = 128          # ... when it has at most this many (request, kv head) pairs


def attention_splits_keys(n_requests: int, num_kv_heads: int, group: int, max_q_len: int, max_context_len: int) -> bool:
    """Whether a step's attention takes the split shape (keys over several blocks plus a combine kernel)."""
    return (max_q_len == 1 and group <= 16 and max_context_len > LONG_CONTEXT
            and n_requests * num_kv_heads <= SPLIT_UP_TO)


def paged_attention_mfma(q: torch.Tensor, k_pages: torch.Tensor, vt_pages: torch.Tensor, block_table: torch.Tensor,
                         q_start: torch.Tensor, context_lens: torch.Tensor, out: torch.Tensor, num_heads: int,
                         scale: float, max_q_len: int, max_context_len: int, window: Optional[int] = None,
                         table_rows: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None,
                         softcap: float = 0.0, slopes: Optional[torch.Tensor] = None,
                         gate: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> torch.Tensor:
    """Matrix-core attention, bfloat16.  k_pages [P, nkv, page_size, d], vt_pages [P, nkv, d, page_size];
    request r owns tokens q_start[r]..q_start[r+1]-1, holds context_lens[r] keys after this step and has row
    ``table_rows[r]`` of ``block_table`` (row r without ``table_rows``).  ``max_q_len`` and ``max_context_len``
    are upper bounds; tokens from q_start[R] on belong to no request, a request may have no token.  A small
    batch of single tokens with long contexts also splits the keys over blocks (and combines).  ``sink`` float [nh]:
    exp(sink[h]) joins the denominator of head h's softmax.  ``softcap``, ``slopes``, ``gate`` and ``out_scale`` as in
    ``paged_attention_generic``."""
    _check(k_pages, "k_pages", torch.bfloat16)
    if sink is not None:
        _check(sink, "sink", torch.float32, (num_heads,))
    if slopes is not None:
        _check(slopes, "slopes", torch.float32, (num_heads,))
    gate_stride = _rows2d(gate, "gate", torch.bfloat16, num_heads) if gate is not None else 0
    if gate is not None and gate.shape[0] != q.shape[0]:
        raise ValueError("gate must have a row per token")
    more = (float(softcap or 0.0), _ptr(slopes), _ptr(gate), gate_stride, float(out_scale))
    P, nkv, page_size, d = k_pages.shape
    _check(vt_pages, "vt_pages", torch.bfloat16, (P, nkv, d, page_size))
    _check(q, "q", torch.bfloat16, contiguous=False)
    N = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < num_heads * d:
        raise ValueError(f"q must be [N, >= {num_heads * d}] with unit stride along rows, got {list(q.shape)}")
    _check(out, "out", torch.bfloat16, (N, num_heads * d))
    _check(block_table, "block_table", torch.int32)
    R = context_lens.numel()
    _check(q_start, "q_start", torch.int32, (R + 1,))
    _check(context_lens, "context_lens", torch.int32, (R,))
    if table_rows is not None:
        _check(table_rows, "table_rows", torch.int32, (R,))
    elif block_table.shape[0] < R:
        raise ValueError(f"the block table has {block_table.shape[0]} rows for {R} requests")
    if num_heads % nkv:
        raise ValueError(f"{num_heads} query heads cannot share {nkv} key/value heads")
    if max_q_len < 1 or max_context_len < max_q_len or max_context_len > block_table.shape[1] * page_size:
        raise ValueError(f"max_q_len {max_q_len} / max_context_len {max_context_len} do not fit a table of "
                         f"{block_table.shape[1]} pages of {page_size}")
    q_stride = q.stride(0) if N > 1 else q.shape[1]
    if attention_splits_keys(R, nkv, num_heads // nkv, max_q_len, max_context_len):
        # a launch constant of the batch size and of the longest context the step is made for (in a captured
        # graph: the cache's capacity, so that the graph stays valid as contexts grow): every request spreads
        # its own key blocks over the splits inside the kernel
        # (measured with contexts of 128 to 4,352 keys: 64 requests x 2 kv heads 30.6 us unsplit, 23.8 in 4 splits;
        # 32 x 2: 29.8, 20.7 in 4, 15.4 in 8; 16 x 4 of 128 dims: 50.7, 23.3 in 8; 8 x 2 at 7,600 keys: 45.6, 13.3
        # in 16, 13.1 in 32).  Contexts of tens of thousands of keys may take more splits, as far as the blocks
        # allow (one request of 100,000 keys, two kv heads: 61 us in 16 splits, 24.4 in 64, 23.4 in 128, 27 in 256).
        most = MAX_SPLITS * (1 if max_context_len <= 16384 else (2 if max_context_len <= 65536 else 8))
        n_splits = max(1, min(most, SPLIT_BLOCKS // max(1, R * nkv)))
        part_o = torch.empty((R, num_heads, n_splits, d), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((R, num_heads, n_splits, 2), dtype=torch.float32, device=q.device)
        _call("ms_paged_attention_mfma_decode", q.data_ptr(), q_stride, k_pages.data_ptr(), vt_pages.data_ptr(),
              block_table.data_ptr(), block_table.shape[1], _ptr(table_rows), q_start.data_ptr(), context_lens.data_ptr(),
              out.data_ptr(), num_heads * d, part_o.data_ptr(), part_ml.data_ptr(), R, num_heads, nkv, d, page_size, float(scale),
              int(window or 0), MIN_BLOCKS_PER_SPLIT, n_splits, _ptr(sink), *more, _stream())
    else:
        _call("ms_paged_attention_mfma", q.data_ptr(), q_stride, k_pages.data_ptr(), vt_pages.data_ptr(),
              block_table.data_ptr(), block_table.shape[1], _ptr(table_rows), q_start.data_ptr(), context_lens.data_ptr(),
              out.data_ptr(), num_heads * d, R, N, max_q_len, num_heads, nkv, d, page_size, float(scale), int(window or 0),
              _ptr(sink), *more, _stream())
    return out


def sample(logits: torch.Tensor, out: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
           seeds: Optional[torch.Tensor] = None, draw_index: Optional[torch.Tensor] = None,
           use_top_k: bool = True, use_top_p: bool = True) -> torch.Tensor:
    """One token per row of float32 logits [M, V].  Without ``temperature`` (or where it is <= 0) the first
    maximum; else a draw after top-k and top-p, repeatable from (seeds[r], draw_index[r]).  ``use_top_k`` /
    ``use_top_p`` False: the caller knows that no row has a top_k in (0, V) / a top_p below 1, and the kernels
    that look for those thresholds are left out."""
    _check(logits, "logits", torch.float32)
    M, V = logits.shape
    _check(out, "out", torch.int32, (M,))
    if M > 65535:
        raise ValueError("at most 65,535 rows to a call")
    if temperature is None:
        n_chunks = max(1, min(128, V // 1024))
        val = torch.empty((M, n_chunks), dtype=torch.float32, device=logits.device)
        idx = torch.empty((M, n_chunks), dtype=torch.int32, device=logits.device)
        _call("ms_argmax", logits.data_ptr(), V, M, V, val.data_ptr(), idx.data_ptr(), n_chunks, out.data_ptr(), _stream())
        return out
    for t, name, dt in ((temperature, "temperature", torch.float32), (top_k, "top_k", torch.int32),
                        (top_p, "top_p", torch.float32), (seeds, "seeds", torch.int64),
                        (draw_index, "draw_index", torch.int32)):
        if t is not None:
            _check(t, name, dt, (M,))
    f = _get("ms_sample_workspace_bytes")
    f.restype = _c_ll
    work = torch.empty(int(f(M)), dtype=torch.uint8, device=logits.device)
    _call("ms_sample", logits.data_ptr(), V, M, V, temperature.data_ptr(), _ptr(top_k), _ptr(top_p), _ptr(seeds),
          _ptr(draw_index), out.data_ptr(), work.data_ptr(), int(use_top_k and top_k is not None),
          int(use_top_p and top_p is not None), _stream())
    return out


def paged_attention(q: torch.Tensor, kv, ctx, out: torch.Tensor, num_heads: int, scale: float,
                    window: Optional[int] = None, sink: Optional[torch.Tensor] = None, softcap: float = 0.0,
                    slopes: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                    out_scale: float = 1.0) -> torch.Tensor:
    """Attention of a step's tokens (``ctx``: its StepContext) over a run's pages (``kv``: its KVView).
    bfloat16 with transposed value pages and a head size the matrix-core kernel has goes there; everything
    else (float32, other head sizes, values of another size than keys, small pages) goes to the generic kernel.
    ``sink`` float [num_heads]: exp(sink[h]) joins the denominator of head h's softmax."""
    d, page_size = kv.k_pages.shape[3], kv.k_pages.shape[2]
    dv = kv.v_pages.shape[2] if kv.v_transposed else kv.v_pages.shape[3]
    if dv != d:
        return paged_attention_generic(q, kv.k_pages, kv.v_pages, kv.block_table, ctx.token_req, ctx.positions, out,
                                       num_heads, scale, window, kv.v_transposed, kv.table_rows, ctx.n_live_tokens, sink,
                                       softcap, slopes, gate, out_scale)
    if q.dtype == torch.bfloat16 and not (kv.v_transposed and attention_mfma_supported(d, page_size)):
        _say_once(("attention", d, page_size),
                  f"bfloat16 attention with head size {d} and pages of {page_size} tokens runs on the vector-ALU kernel: "
                  f"the matrix-core kernel takes head sizes 32, 64 and 128 with pages of a multiple of 16")
    if (q.dtype == torch.bfloat16 and kv.v_transposed and attention_mfma_supported(d, page_size)
            and q.data_ptr() % 16 == 0 and (q.shape[0] == 1 or q.stride(0) % 8 == 0)):
        return paged_attention_mfma(q, kv.k_pages, kv.v_pages, kv.block_table, ctx.q_start, ctx.context_lens, out,
                                    num_heads, scale, ctx.max_q_len, ctx.max_context_len, window, kv.table_rows, sink,
                                    softcap, slopes, gate, out_scale)
    return paged_attention_generic(q, kv.k_pages, kv.v_pages, kv.block_table, ctx.token_req, ctx.positions, out,
                                   num_heads, scale, window, kv.v_transposed, kv.table_rows, ctx.n_live_tokens, sink,
                                   softcap, slopes, gate, out_scale)


# ------------------------------------------------------------------------------------------------ state-carrying mixers
CONV_SUM, CONV_ADD_INPUT, CONV_SILU = 0, 1, 2
MAX_CONV_TAPS = 8


def _rows2d(t: torch.Tensor, name: str, dtype=None, cols=None):
    """A matrix whose rows may be slices of wider rows (unit stride along a row)."""
    _check(t, name, dtype, contiguous=False)
    if t.dim() != 2 or t.stride(1) != 1 or (cols is not None and t.shape[1] != cols):
        raise ValueError(f"{name} must be [rows, {cols if cols is not None else 'columns'}] with unit stride along rows, "
                         f"got {list(t.shape)} strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else t.shape[1]


def short_conv(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, ctx, out: torch.Tensor,
               mode: int = CONV_SUM, update_state: bool = True, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A causal convolution over time on every channel of ``x`` [N, C], for the step ``ctx`` describes:
    out[n] = act(sum_j weight[:, j] * input(t - taps + 1 + j)), the last column meeting the token itself, inputs before a
    request's portion taken from ``state`` [slots, taps - 1, C] (the request's slot; zero at a request's start).
    ``mode``: CONV_SUM, CONV_ADD_INPUT (x + the sum) or CONV_SILU.  With ``update_state`` the state then becomes the
    last taps - 1 inputs of every request of the step.  ``weight`` float [C, taps]; ``bias`` float [C] is added to the sum."""
    N, C = x.shape
    xs = _rows2d(x, "x")
    os_ = _rows2d(out, "out", x.dtype, C)
    if out.shape[0] != N or out.data_ptr() == x.data_ptr():
        raise ValueError("out must be another tensor of x's shape")
    _check(weight, "weight", torch.float32, (C, None))
    taps = weight.shape[1]
    if taps > MAX_CONV_TAPS:
        raise UnsupportedShape(f"the short convolution takes up to {MAX_CONV_TAPS} taps, got {taps}")
    _check(state, "state", x.dtype, (None, max(1, taps - 1), C))
    if bias is not None:
        _check(bias, "bias", torch.float32, (C,))
    R = ctx.num_requests
    _check(ctx.token_req, "token_req", torch.int32, (N,))
    _check(ctx.q_start, "q_start", torch.int32, (R + 1,))
    _check(ctx.state_slots, "state_slots", torch.int32, (R,))
    _call("ms_short_conv", x.data_ptr(), xs, weight.data_ptr(), _ptr(bias), state.data_ptr(), ctx.token_req.data_ptr(),
          ctx.q_start.data_ptr(), ctx.state_slots.data_ptr(), _ptr(ctx.n_live_tokens), out.data_ptr(), os_, N, R, C, taps,
          mode, int(update_state), int(getattr(ctx, "max_q_len", 0) == 1), _code(x.dtype), _stream())
    return out


def gated_delta(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a: torch.Tensor, b: torch.Tensor, A_log: torch.Tensor,
                dt_bias: torch.Tensor, state: torch.Tensor, ctx, out: torch.Tensor, heads: int, kv_heads: int, dim: int,
                vdim: int, decay_per_channel: bool = True) -> torch.Tensor:
    """The gated delta rule over the step's portions, from and into ``state`` float [slots, heads, dim, vdim]:
    per head and token  S <- g * S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q  with q, k made unit vectors
    (q also times dim^-1/2), beta = sigmoid(b), g = exp(-exp(A_log) * softplus(a + dt_bias)).  q, k [N, kv_heads * dim],
    v [N, heads * vdim] and b [N, heads] are row slices with one row stride for q, k, v; a float [N, heads * dim] with
    dt_bias [heads * dim] (a decay per head and key channel) or a float [N, heads] with dt_bias [heads] (a decay per
    head); out float [N, heads * vdim]."""
    N = q.shape[0]
    sq = _rows2d(q, "q", None, kv_heads * dim)
    sk = _rows2d(k, "k", q.dtype, kv_heads * dim)
    sv = _rows2d(v, "v", q.dtype, heads * vdim)
    if not (sq == sk == sv) and N > 1:
        raise ValueError("q, k and v must be slices of rows of one width")
    sb = _rows2d(b, "b", q.dtype, heads)
    _check(A_log, "A_log", torch.float32, (heads,))
    per_channel = bool(decay_per_channel)
    _check(a, "a", torch.float32, (N, heads * dim if per_channel else heads))
    _check(dt_bias, "dt_bias", torch.float32, (heads * dim if per_channel else heads,))
    _check(state, "state", torch.float32, (None, heads, dim, vdim))
    _check(out, "out", torch.float32, (N, heads * vdim))
    R = ctx.num_requests
    _check(ctx.q_start, "q_start", torch.int32, (R + 1,))
    _check(ctx.state_slots, "state_slots", torch.int32, (R,))
    if heads % kv_heads:
        raise ValueError(f"{heads} heads cannot share {kv_heads} query/key heads")
    _call("ms_gated_delta", q.data_ptr(), k.data_ptr(), v.data_ptr(), sq, a.data_ptr(), int(per_channel), b.data_ptr(), sb,
          A_log.data_ptr(),
          dt_bias.data_ptr(), state.data_ptr(), ctx.q_start.data_ptr(), ctx.state_slots.data_ptr(), out.data_ptr(), R,
          heads, kv_heads, dim, vdim, int(getattr(ctx, "max_q_len", 0) == 1), _code(q.dtype), _stream())
    return out


def gated_head_norm(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, out: torch.Tensor, heads: int, vdim: int,
                    eps: float, gate_act: str = "sigmoid", scale: float = 1.0) -> torch.Tensor:
    """out[n, h] = scale * o[n, h] / sqrt(mean(o[n, h]^2) + eps) * weight * act(gate[n, h]), act "sigmoid" or "silu";
    o float [N, heads * vdim]; weight float [vdim], shared by the heads, or [heads * vdim], every head its own."""
    if gate_act not in ("sigmoid", "silu"):
        raise ValueError(f"the read-out's gate is 'sigmoid' or 'silu', not {gate_act!r}")
    N = o.shape[0]
    _check(o, "o", torch.float32, (N, heads * vdim))
    per_head = weight.numel() == heads * vdim and heads > 1
    _check(weight, "weight", torch.float32, (heads * vdim if per_head else vdim,))
    gs = _rows2d(gate, "gate", out.dtype, heads * vdim)
    _check(out, "out", None, (N, heads * vdim))
    _call("ms_gated_head_norm", o.data_ptr(), weight.data_ptr(), gate.data_ptr(), gs, out.data_ptr(), N, heads, vdim,
          float(eps), int(gate_act == "silu"), int(per_head), float(scale), _code(out.dtype), _stream())
    return out


DECAY_SIGMOID_ROOT, DECAY_DOUBLE_EXP = 0, 1
RECURRENCE_STRETCH = 128             # tokens of a long portion that one block walks when the portion is spread over blocks
RECURRENCE_SPREAD_FROM = 256         # the portion length from which that pays
RECURRENCE_SCRATCH_BYTES = 1 << 29   # the most scratch a spread step may take


def decay_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, z: torch.Tensor, z_bias: Optional[torch.Tensor],
                     state: torch.Tensor, ctx, out: torch.Tensor, heads: int, dim: int, vdim: int, decay: int,
                     tau: float = 1.0, bonus: Optional[torch.Tensor] = None, q_scale: float = 1.0) -> torch.Tensor:
    """A recurrence with a decay per head and key channel over the step's portions, from and into ``state`` float
    [slots, heads, dim, vdim]: per head and token  S <- diag(w) S + k v^T  and  o = S^T (q_scale q)  read after the write;
    with ``bonus`` u float [heads * dim] the read comes first and weights the current token:
    o = (S + diag(u) k v^T)^T (q_scale q), then the write.  The decay is made from z float [N, heads * dim] (+ ``z_bias``
    float [heads * dim]): DECAY_SIGMOID_ROOT: w = sigmoid(z)^(1 / tau); DECAY_DOUBLE_EXP: w = exp(-exp(z)).  q, k
    [N, heads * dim] and v [N, heads * vdim] may be row slices; out float [N, heads * vdim].  A step with long portions
    (``ctx.max_q_len``, an upper bound) cuts them into stretches that run side by side and are joined through the
    recurrence's linearity, in two launches; the float sums then associate differently, within rounding."""
    N = q.shape[0]
    sq = _rows2d(q, "q", None, heads * dim)
    sk = _rows2d(k, "k", q.dtype, heads * dim)
    sv = _rows2d(v, "v", q.dtype, heads * vdim)
    if k.shape[0] != N or v.shape[0] != N:
        raise ValueError("q, k and v must have a row per token")
    _check(z, "z", torch.float32, (N, heads * dim))
    if z_bias is not None:
        _check(z_bias, "z_bias", torch.float32, (heads * dim,))
    if bonus is not None:
        _check(bonus, "bonus", torch.float32, (heads * dim,))
    if decay not in (DECAY_SIGMOID_ROOT, DECAY_DOUBLE_EXP):
        raise ValueError("decay is DECAY_SIGMOID_ROOT or DECAY_DOUBLE_EXP")
    if decay == DECAY_SIGMOID_ROOT and not tau > 0:
        raise ValueError("tau must be positive")
    _check(state, "state", torch.float32, (None, heads, dim, vdim))
    _check(out, "out", torch.float32, (N, heads * vdim))
    R = ctx.num_requests
    _check(ctx.q_start, "q_start", torch.int32, (R + 1,))
    _check(ctx.state_slots, "state_slots", torch.int32, (R,))
    longest = min(int(getattr(ctx, "max_q_len", 0) or 0), N)
    stretches, pair_a, pair_b = 1, None, None
    if longest >= RECURRENCE_SPREAD_FROM:
        stretches = -(-longest // RECURRENCE_STRETCH)
        if R * stretches > 65535 or 4 * R * stretches * heads * dim * (vdim + 1) > RECURRENCE_SCRATCH_BYTES:
            stretches = 1
        else:
            pair_a = torch.empty((R, stretches, heads, dim), dtype=torch.float32, device=q.device)
            pair_b = torch.empty((R, stretches, heads, dim, vdim), dtype=torch.float32, device=q.device)
    _call("ms_decay_recurrence", q.data_ptr(), k.data_ptr(), v.data_ptr(), sq, sk, sv, z.data_ptr(), _ptr(z_bias), int(decay),
          1.0 / float(tau), _ptr(bonus), float(q_scale), state.data_ptr(), ctx.q_start.data_ptr(), ctx.state_slots.data_ptr(),
          out.data_ptr(), R, heads, dim, vdim, RECURRENCE_STRETCH, stretches, _ptr(pair_a), _ptr(pair_b), _code(q.dtype),
          _stream())
    return out


def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, ctx, out: torch.Tensor) -> torch.Tensor:
    """out[m, n] = h[n] + (h'[n] - h[n]) o mu[m] for the step ``ctx`` describes, h' the previous token's row of h: the row
    before within a portion, ``state`` [slots, 1, W] (the request's slot; zero at a request's start) for a portion's first
    token.  The state then becomes the last row of every request's portion.  mu float [M, W]; out [M, N, W] of h's type."""
    N, W = h.shape
    hs = _rows2d(h, "h")
    _check(mu, "mu", torch.float32, (None, W))
    M = mu.shape[0]
    _check(state, "state", h.dtype, (None, 1, W))
    _check(out, "out", h.dtype, (M, N, W))
    R = ctx.num_requests
    _check(ctx.token_req, "token_req", torch.int32, (N,))
    _check(ctx.q_start, "q_start", torch.int32, (R + 1,))
    _check(ctx.state_slots, "state_slots", torch.int32, (R,))
    _call("ms_token_shift", h.data_ptr(), hs, mu.data_ptr(), state.data_ptr(), ctx.token_req.data_ptr(), ctx.q_start.data_ptr(),
          ctx.state_slots.data_ptr(), _ptr(ctx.n_live_tokens), out.data_ptr(), N, R, W, M, _code(h.dtype), _stream())
    return out


def pair_sum(x: torch.Tensor, a: torch.Tensor, b: torch.Tensor, scale_a: float = 1.0, scale_b: float = 1.0,
             norm_a: Optional[torch.Tensor] = None, norm_b: Optional[torch.Tensor] = None, eps: float = 0.0) -> torch.Tensor:
    """x[n] += scale_a f(a[n]) + scale_b g(b[n]), in place on the float residual stream; f is the identity, or with
    ``norm_a`` (float [W]) the row divided by its root mean square (eps inside the root) times that weight; g likewise."""
    _check(x, "x", torch.float32)
    N, W = x.shape
    _check(a, "a", None, (N, W))
    _check(b, "b", a.dtype, (N, W))
    for w, name in ((norm_a, "norm_a"), (norm_b, "norm_b")):
        if w is not None:
            _check(w, name, torch.float32, (W,))
    _call("ms_pair_sum", a.data_ptr(), b.data_ptr(), float(scale_a), float(scale_b), _ptr(norm_a), _ptr(norm_b), float(eps),
          x.data_ptr(), N, W, _code(a.dtype), _stream())
    return x


def tanh_(x: torch.Tensor) -> torch.Tensor:
    """x <- tanh(x), in place (computed in float, rounded once)."""
    _check(x, "x")
    _call("ms_tanh", x.data_ptr(), x.numel(), _code(x.dtype), _stream())
    return x


def concat_rows(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[n] = [a[n] | b[n]] in out's type; a [N, Wa] and b [N, Wb] float."""
    _check(a, "a", torch.float32)
    _check(b, "b", torch.float32, (a.shape[0], None))
    _check(out, "out", None, (a.shape[0], a.shape[1] + b.shape[1]))
    _call("ms_concat_rows", a.data_ptr(), b.data_ptr(), out.data_ptr(), a.shape[0], a.shape[1], b.shape[1], _code(out.dtype),
          _stream())
    return out


def xielu(x: torch.Tensor, pq: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z/2; z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2, with pq = (p, q) float [2]."""
    _check(x, "x")
    _check(pq, "pq", torch.float32, (2,))
    _check(out, "out", x.dtype, tuple(x.shape))
    _call("ms_xielu", x.data_ptr(), pq.data_ptr(), out.data_ptr(), x.numel(), _code(x.dtype), _stream())
    return out


# ------------------------------------------------------------------------------------------------ attention through a latent
def _heads3d(t: torch.Tensor, name: str, dtype=None):
    _check(t, name, dtype, contiguous=False)
    if t.dim() != 3 or t.stride(2) != 1:
        raise ValueError(f"{name} must be [tokens, heads, width] with unit stride along the width, got {list(t.shape)} "
                         f"strides {t.stride()}")
    return t.stride(0), t.stride(1)


def head_matmul(x: torch.Tensor, m: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n, h, :] = x[n, h, :] @ m[h] (* sigmoid(gate[n, h, :])).  x [N, H, I] and out [N, H, J] may be views with any
    token and head strides; m [H, I, J] contiguous; gate [N, H * J] rows."""
    N, H, I = x.shape
    xt, xh = _heads3d(x, "x")
    _check(m, "m", x.dtype, (H, I, None))
    J = m.shape[2]
    ot, oh = _heads3d(out, "out")
    if tuple(out.shape) != (N, H, J):
        raise ValueError(f"out must be {[N, H, J]}, got {list(out.shape)}")
    gs = 0
    if gate is not None:
        gs = _rows2d(gate, "gate", x.dtype, H * J)
    _call("ms_head_matmul", x.data_ptr(), xt, xh, m.data_ptr(), out.data_ptr(), ot, oh, _ptr(gate), gs, N, H, I, J,
          _code(x.dtype), _code(out.dtype), _stream())
    return out


def rms_norm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> torch.Tensor:
    """out[n] = x[n] / sqrt(mean(x[n]^2) + eps) * weight for rows of an activation (row slices are fine)."""
    N, C = x.shape
    xs = _rows2d(x, "x")
    os_ = _rows2d(out, "out", x.dtype, C)
    _check(weight, "weight", torch.float32, (C,))
    _call("ms_rms_norm_rows", x.data_ptr(), xs, weight.data_ptr(), out.data_ptr(), os_, N, C, float(eps), _code(x.dtype),
          _stream())
    return out


def rotary_pairs(src: torch.Tensor, dst: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """dst[n, h] = src[n, h] with its first 2 * len(inv_freq) entries turned, entry 2i with entry 2i + 1, by
    float(positions[n]) * inv_freq[i]; the rest is copied.  src, dst [N, H, width] views (dst may be src)."""
    N, H, width = src.shape
    st, sh = _heads3d(src, "src")
    dt, dh = _heads3d(dst, "dst", src.dtype)
    if tuple(dst.shape) != (N, H, width):
        raise ValueError("dst must have src's shape")
    _check(positions, "positions", torch.int32, (N,))
    _check(inv_freq, "inv_freq", torch.float32)
    dims = 2 * inv_freq.numel()
    if dims > width:
        raise ValueError(f"{dims} rotated entries do not fit a width of {width}")
    _call("ms_rotary_pairs", src.data_ptr(), st, sh, dst.data_ptr(), dt, dh, positions.data_ptr(), inv_freq.data_ptr(), N, H,
          width, dims, _code(src.dtype), _stream())
    return dst


launches = {}     # how often a dispatcher below chose a kernel that tests want to see chosen: name -> times


def latent_mfma_sizes(C: int, R: int) -> bool:
    """Whether the matrix-core attention over latents has a variant for a latent of C and a rotated part of R entries
    (the library's ms_latent_attention_mfma_supported says the same, and more about pages)."""
    return C in (128, 256, 512) and R in (32, 64)


def latent_kv_store(kv: torch.Tensor, norm_weight: torch.Tensor, eps: float, positions: torch.Tensor, inv_freq: torch.Tensor,
                    slot_mapping: torch.Tensor, c_pages: torch.Tensor, r_pages: torch.Tensor,
                    ct_pages: Optional[torch.Tensor] = None) -> None:
    """kv [N, C + R]: the RMS norm of its first C columns (times ``norm_weight``) goes to ``c_pages`` [P, 1, page, C], its
    last R columns, turned pair by pair, to ``r_pages`` [P, 1, page, R], at ``slot_mapping`` (< 0: not stored).
    ``ct_pages`` [P, 1, C, page], if given, takes the same latents transposed."""
    N = kv.shape[0]
    _check(c_pages, "c_pages", kv.dtype, (None, 1, None, None))
    C = c_pages.shape[3]
    _check(r_pages, "r_pages", kv.dtype, (c_pages.shape[0], 1, c_pages.shape[2], None))
    R = r_pages.shape[3]
    if ct_pages is not None:
        _check(ct_pages, "ct_pages", kv.dtype, (c_pages.shape[0], 1, C, c_pages.shape[2]))
    ks = _rows2d(kv, "kv", None, C + R)
    _check(norm_weight, "norm_weight", torch.float32, (C,))
    _check(positions, "positions", torch.int32, (N,))
    _check(slot_mapping, "slot_mapping", torch.int32, (N,))
    _check(inv_freq, "inv_freq", torch.float32)
    _call("ms_latent_kv_store", kv.data_ptr(), ks, norm_weight.data_ptr(), float(eps), positions.data_ptr(),
          inv_freq.data_ptr(), slot_mapping.data_ptr(), c_pages.data_ptr(), r_pages.data_ptr(), _ptr(ct_pages),
          c_pages.shape[2], N, C, R, 2 * inv_freq.numel(), _code(kv.dtype), _stream())


def latent_attention(q: torch.Tensor, kv, ctx, out: torch.Tensor, scale: float, window: Optional[int] = None,
                     sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n, h] = sum_j p_j c_j over the keys j visible to token n (the last ``window`` up to itself), with
    p = exp(s_j) / (sum_i exp(s_i) + exp(sink[h])) and s_j = scale * q[n, h] . [c_j ; kr_j].  q [N, H, C + R] and out
    [N, H, C] views; ``kv``: a KVView whose pages are "c" [P, 1, page, C] and "kr" [P, 1, page, R]."""
    c_pages, r_pages = kv.pages["c"], kv.pages["kr"]
    _check(c_pages, "c_pages", q.dtype, (None, 1, None, None))
    P, _, page_size, C = c_pages.shape
    _check(r_pages, "r_pages", q.dtype, (P, 1, page_size, None))
    R = r_pages.shape[3]
    N, H, width = q.shape
    if width != C + R:
        raise ValueError(f"queries of width {width} against keys of {C} + {R}")
    qt, qh = _heads3d(q, "q")
    ot, oh = _heads3d(out, "out", q.dtype)
    if tuple(out.shape) != (N, H, C):
        raise ValueError(f"out must be {[N, H, C]}, got {list(out.shape)}")
    _check(kv.block_table, "block_table", torch.int32)
    _check(ctx.token_req, "token_req", torch.int32, (N,))
    _check(ctx.positions, "positions", torch.int32, (N,))
    if kv.table_rows is not None:
        _check(kv.table_rows, "table_rows", torch.int32)
    if sink is not None:
        _check(sink, "sink", torch.float32, (H,))
    ct_pages = kv.pages.get("ct")
    if (q.dtype == torch.bfloat16 and ct_pages is not None and kv.transposed.get("ct") and latent_mfma_sizes(C, R)
            and page_size % 16 == 0 and qt % 8 == 0 and qh % 8 == 0 and ot % 4 == 0 and oh % 4 == 0
            and q.data_ptr() % 16 == 0 and out.data_ptr() % 8 == 0 and getattr(ctx, "max_q_len", 0) > 0):
        # the matrix-core kernel: it reads the latents' transposed copy as the operand of the weighted sum
        launches["latent_attention_mfma"] = launches.get("latent_attention_mfma", 0) + 1
        _check(ct_pages, "ct_pages", q.dtype, (P, 1, C, page_size))
        Rq = ctx.num_requests
        _check(ctx.q_start, "q_start", torch.int32, (Rq + 1,))
        _check(ctx.context_lens, "context_lens", torch.int32, (Rq,))
        _call("ms_latent_attention_mfma", q.data_ptr(), qt, qh, c_pages.data_ptr(), r_pages.data_ptr(), ct_pages.data_ptr(),
              kv.block_table.data_ptr(), kv.block_table.shape[1], _ptr(kv.table_rows), ctx.q_start.data_ptr(),
              ctx.context_lens.data_ptr(), _ptr(sink), out.data_ptr(), ot, oh, Rq, ctx.max_q_len, H, C, R, page_size, P,
              float(scale), int(window or 0), _stream())
        return out
    _call("ms_latent_attention", q.data_ptr(), qt, qh, c_pages.data_ptr(), r_pages.data_ptr(), kv.block_table.data_ptr(),
          kv.block_table.shape[1], _ptr(kv.table_rows), _ptr(ctx.n_live_tokens), ctx.token_req.data_ptr(),
          ctx.positions.data_ptr(), _ptr(sink), out.data_ptr(), ot, oh, N, H, C, R, page_size, P, float(scale),
          int(window or 0), _code(q.dtype), _stream())
    return out


# ------------------------------------------------------------------------------------------------ norms after a sublayer
def rms_norm_add(y: torch.Tensor, w_post: torch.Tensor, eps_post: float, x: torch.Tensor,
                 w_next: Optional[torch.Tensor] = None, eps_next: float = 0.0,
                 out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x += w_post * y / sqrt(mean(y^2) + eps_post), in place on the float residual stream x [N, H]; y [N, H] (rows may be
    slices of wider rows) is a sublayer's output.  With ``out`` [N, H] also out = w_next * x / sqrt(mean(x^2) + eps_next),
    the norm the next sublayer reads, from the same pass."""
    _check(x, "x", torch.float32)
    N, H = x.shape
    ys = _rows2d(y, "y", None, H)
    if y.shape[0] != N:
        raise ValueError(f"y has {y.shape[0]} rows, x {N}")
    _check(w_post, "w_post", torch.float32, (H,))
    ocode = 0
    if out is not None:
        _check(out, "out", None, (N, H))
        _check(w_next, "w_next", torch.float32, (H,))
        ocode = _code(out.dtype)
    _call("ms_rms_norm_add", y.data_ptr(), ys, _code(y.dtype), w_post.data_ptr(), float(eps_post), x.data_ptr(),
          _ptr(w_next) if out is not None else None, float(eps_next), _ptr(out), ocode, N, H, _stream())
    return out


def add_rows(x: torch.Tensor, kept: Optional[torch.Tensor] = None, vec: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[n] += kept[n] + vec, in place; x and kept float [N, H], vec float [H]; either addend may be left out."""
    _check(x, "x", torch.float32)
    N, H = x.shape
    if kept is not None:
        _check(kept, "kept", torch.float32, (N, H))
    if vec is not None:
        _check(vec, "vec", torch.float32, (H,))
    if kept is None and vec is None:
        return x
    _call("ms_add_rows", x.data_ptr(), _ptr(kept), _ptr(vec), N, H, _stream())
    return x


def qk_norm_store(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                  q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                  positions: Optional[torch.Tensor] = None, coef: float = 0.0, every: int = 1,
                  slot_mapping: Optional[torch.Tensor] = None, k_pages: Optional[torch.Tensor] = None,
                  v_pages: Optional[torch.Tensor] = None, v_transposed: bool = False, unit_norm: bool = False,
                  inv_freq: Optional[torch.Tensor] = None, rot_dim: int = 0) -> torch.Tensor:
    """In place on ``qkv`` [N, nh d + nkv d + nkv dv]: the RMS norm of every q and k head with the weights [d] (None: no
    norm, or with ``unit_norm`` the division by the root mean square alone), q of the token at position p times
    1 + coef * ln(floor((p + 1) / every) + 1); with ``rot_dim`` > 0 entry i and entry i + rot_dim / 2 of every q and k head
    then turn by position * inv_freq[i] (float [rot_dim / 2]); then k and v go into the pages
    ([P, nkv, page, d] and [P, nkv, page, dv], or values [P, nkv, dv, page] with ``v_transposed``) at ``slot_mapping``."""
    width = (num_heads + num_kv_heads) * head_dim + num_kv_heads * value_dim
    stride = _rows2d(qkv, "qkv", None, width)
    N = qkv.shape[0]
    for w, name in ((q_weight, "q_weight"), (k_weight, "k_weight")):
        if w is not None:
            _check(w, name, torch.float32, (head_dim,))
    if coef:
        _check(positions, "positions", torch.int32, (N,))
        if every <= 0:
            raise ValueError("the query temperature's period must be positive")
    if rot_dim:
        if rot_dim % 2 or not 0 < rot_dim <= head_dim:
            raise ValueError(f"{rot_dim} rotated entries must be even and within the head's {head_dim}")
        _check(positions, "positions", torch.int32, (N,))
        _check(inv_freq, "inv_freq", torch.float32, (rot_dim // 2,))
    page_size = 0
    if k_pages is not None:
        _check(k_pages, "k_pages", qkv.dtype, (None, num_kv_heads, None, head_dim))
        page_size = k_pages.shape[2]
        _check(v_pages, "v_pages", qkv.dtype, _v_shape(k_pages, v_transposed, value_dim))
        _check(slot_mapping, "slot_mapping", torch.int32, (N,))
    _call("ms_qk_norm_store", qkv.data_ptr(), stride, _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(positions), float(coef),
          int(every), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages), N, num_heads, num_kv_heads, head_dim, value_dim,
          page_size, int(bool(v_transposed)), int(bool(unit_norm)), _ptr(inv_freq) if rot_dim else None, int(rot_dim),
          _code(qkv.dtype), _stream())
    return qkv


# ------------------------------------------------------------------------------------------------ selective scan
SCAN_MAX_STATES = 256


def selective_scan(x: torch.Tensor, dt_in: torch.Tensor, dt_bias: torch.Tensor, A: torch.Tensor, B: torch.Tensor,
                   C: torch.Tensor, D: torch.Tensor, z: torch.Tensor, state: torch.Tensor, ctx, out: torch.Tensor) -> torch.Tensor:
    """The selective scan over the step's portions, from and into ``state`` float [slots, I, S]: per channel c and state n
    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;  y_c = sum_n S[c, n] C_n + D_c x_c;  out = y * silu(z), with
    dt = softplus(dt_in + dt_bias).  x, z [N, I] and B, C [N, S] are row slices (B and C of one row stride); dt_in float
    [N, I]; A float [I, S]; D, dt_bias float [I]; out [N, I]."""
    N, I = x.shape
    xs = _rows2d(x, "x")
    zs = _rows2d(z, "z", x.dtype, I)
    S = A.shape[1]
    bs = _rows2d(B, "B", x.dtype, S)
    cs = _rows2d(C, "C", x.dtype, S)
    if bs != cs and N > 1:
        raise ValueError("B and C must be slices of rows of one width")
    os_ = _rows2d(out, "out", x.dtype, I)
    if z.shape[0] != N or B.shape[0] != N or C.shape[0] != N or out.shape[0] != N:
        raise ValueError("x, z, B, C and out have one row per token")
    _check(dt_in, "dt_in", torch.float32, (N, I))
    _check(dt_bias, "dt_bias", torch.float32, (I,))
    _check(A, "A", torch.float32, (I, S))
    _check(D, "D", torch.float32, (I,))
    _check(state, "state", torch.float32, (None, I, S))
    R = ctx.num_requests
    _check(ctx.q_start, "q_start", torch.int32, (R + 1,))
    _check(ctx.state_slots, "state_slots", torch.int32, (R,))
    _call("ms_selective_scan", x.data_ptr(), xs, dt_in.data_ptr(), dt_bias.data_ptr(), A.data_ptr(), B.data_ptr(), C.data_ptr(),
          bs, D.data_ptr(), z.data_ptr(), zs, state.data_ptr(), ctx.q_start.data_ptr(), ctx.state_slots.data_ptr(),
          out.data_ptr(), os_, R, I, S, _code(x.dtype), _stream())
    return out


# ------------------------------------------------------------------------------------------------ routed experts
ROUTE_MAX_OUTPUTS, ROUTE_MAX_TOP = 1024, 32


def gelu(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = x/2 (1 + erf(x / sqrt 2)), the exact gelu, worked out in float."""
    _check(x, "x")
    _check(out, "out", x.dtype, tuple(x.shape))
    _call("ms_gelu", x.data_ptr(), out.data_ptr(), x.numel(), _code(x.dtype), _stream())
    return out


def moe_route(logits: torch.Tensor, correction: Optional[torch.Tensor], top: int, n_out: Optional[int] = None,
              scores: str = "softmax"):
    """Scores = softmax(logits[:, :n_out]) (``scores`` "sigmoid": every logit's own sigmoid); the ``top`` largest of
    scores + correction are chosen (the lower index on a tie).  Returns (ids int32 [N, top], their scores float [N, top]).
    logits float [N, >= n_out]."""
    if scores not in ("softmax", "sigmoid"):
        raise ValueError(f"router scores are 'softmax' or 'sigmoid', not {scores!r}")
    ld = _rows2d(logits, "logits", torch.float32)
    N = logits.shape[0]
    n_out = logits.shape[1] if n_out is None else n_out
    if not 0 < top <= n_out <= logits.shape[1]:
        raise ValueError(f"top {top} of {n_out} outputs in rows of {logits.shape[1]}")
    if correction is not None:
        _check(correction, "correction", torch.float32, (n_out,))
    ids = torch.empty((N, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((N, top), dtype=torch.float32, device=logits.device)
    _call("ms_moe_route", logits.data_ptr(), ld, _ptr(correction), N, n_out, top, ids.data_ptr(), weights.data_ptr(),
          int(scores == "sigmoid"), _stream())
    return ids, weights


def moe_tile_rows() -> int:
    return int(_get("ms_moe_tile_rows")())


def moe_wide_tile_rows() -> int:
    return int(_get("ms_moe_wide_tile_rows")())


def moe_widest_tile_rows() -> int:
    return int(_get("ms_gemm_tiled_grouped_rows")())


def moe_tile_choice(n_items: int, n_experts: int, sizes, dtype: torch.dtype) -> int:
    """The rows of a tile for the grouped products of ``n_items`` rows over ``n_experts`` experts whose matrices have
    the row lengths ``sizes``.  An expert's matrix is read once for every tile of its rows, so wider tiles read less:
    on the matrix cores (bfloat16), once an expert has a wide tile's rows on average (so that most tiles are full),
    ``moe_widest_tile_rows()`` where every size is a multiple of 64 (half-empty tiles cost matrix-core time that the
    product, bound by the bytes it moves, has to spare), else
    ``moe_wide_tile_rows()`` where every size is a multiple of 32; ``moe_tile_rows()`` otherwise (a decode step: the
    chosen experts' matrices stream once)."""
    if dtype == torch.bfloat16 and n_items >= moe_wide_tile_rows() * n_experts:
        if all(k % 64 == 0 for k in sizes):
            return moe_widest_tile_rows()
        if all(k % 32 == 0 for k in sizes):
            return moe_wide_tile_rows()
    return moe_tile_rows()


def moe_align(ids: torch.Tensor, n_experts: int, tile: Optional[int] = None):
    """Groups the rows (token, choice) of ``ids`` [N, top] by expert into tiles of ``tile`` rows (``moe_tile_rows()``,
    the default, ``moe_wide_tile_rows()`` or ``moe_widest_tile_rows()``) of one expert each.  Returns (rows int32 [tiles * tile]: the flat index n * top + j of every
    row or -1, tile_expert int32 [tiles]: the tile's expert or -1).  Choices >= n_experts (experts without weights) take
    no row.  The number of tiles depends on the sizes alone."""
    _check(ids, "ids", torch.int32)
    n_items = ids.numel()
    tile = moe_tile_rows() if tile is None else int(tile)
    if tile not in (moe_tile_rows(), moe_wide_tile_rows(), moe_widest_tile_rows()):
        raise ValueError(f"tiles have {moe_tile_rows()}, {moe_wide_tile_rows()} or {moe_widest_tile_rows()} rows, not {tile}")
    tiles = (n_items + n_experts * (tile - 1) + tile - 1) // tile
    rows = torch.empty(tiles * tile, dtype=torch.int32, device=ids.device)
    tile_expert = torch.empty(tiles, dtype=torch.int32, device=ids.device)
    _call("ms_moe_align", ids.data_ptr(), n_items, n_experts, tile, tiles, rows.data_ptr(), tile_expert.data_ptr(), _stream())
    return rows, tile_expert


def grouped_gemm(a: torch.Tensor, w: torch.Tensor, rows: torch.Tensor, tile_expert: torch.Tensor, out: torch.Tensor,
                 gather_div: int = 0, scatter: bool = False, act: Optional[str] = None) -> torch.Tensor:
    """For every tile with an expert e and every row of it (flat position p, item = rows[p] >= 0):
    out[item if scatter else p] = act(a[item // gather_div if gather_div else p] @ w[e].T); w [experts, n_out, K]; float
    accumulation in the order of K.  ``act``: None or "gelu".  The tiles' size is read off ``rows`` and ``tile_expert``
    (``moe_align``'s); bfloat16 with K a multiple of 32 runs on the matrix cores (the widest tiles: a multiple of 64),
    everything else on the vector ALUs (tiles of ``moe_tile_rows()`` rows only)."""
    _check(w, "w", a.dtype)
    if w.dim() != 3:
        raise ValueError("w must be [experts, out features, in features]")
    E, n_out, K = w.shape
    a_stride = _rows2d(a, "a", None, K)
    o_stride = _rows2d(out, "out", None, n_out)
    _check(tile_expert, "tile_expert", torch.int32)
    tiles = tile_expert.numel()
    _check(rows, "rows", torch.int32)
    tile = rows.numel() // max(1, tiles)
    if tile * tiles != rows.numel() or tile not in (moe_tile_rows(), moe_wide_tile_rows(), moe_widest_tile_rows()):
        raise ValueError(f"{rows.numel()} rows do not make {tiles} tiles of {moe_tile_rows()}, {moe_wide_tile_rows()} or "
                         f"{moe_widest_tile_rows()}")
    if not gather_div and a.shape[0] < tiles * tile:
        raise ValueError("a must hold a row for every row of every tile")
    if not scatter and out.shape[0] < tiles * tile:
        raise ValueError("out must hold a row for every row of every tile")
    if act not in (None, "gelu"):
        raise ValueError(f"no activation {act!r} here")
    _call("ms_grouped_gemm", a.data_ptr(), a_stride, w.data_ptr(), rows.data_ptr(), tile_expert.data_ptr(), out.data_ptr(),
          o_stride, tiles, tile, n_out, K, int(gather_div), int(scatter), int(act == "gelu"), _code(a.dtype),
          _code(out.dtype), _stream())
    return out


def moe_combine(part: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, h: torch.Tensor, n_experts: int,
                out: torch.Tensor, shared: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n] = sum_j weights[n, j] * (part[n * top + j] if ids[n, j] < n_experts else h[n]) + sigmoid(gate[n]) * shared[n].
    part float [N * top, H]; h [N, H]; shared [N, H] (h's type or float) with gate float [N] (a column of a wider matrix
    is fine); out float [N, H]."""
    N, top = ids.shape
    _check(ids, "ids", torch.int32)
    if weights is not None:      # None: every choice weighs 1
        _check(weights, "weights", torch.float32, (N, top))
    H = out.shape[1]
    _check(part, "part", torch.float32, (N * top, H))
    hs = _rows2d(h, "h", None, H)
    _check(out, "out", torch.float32, (N, H))
    gs, scode = 0, 0
    if shared is not None:
        _check(shared, "shared", None, (N, H))
        scode = _code(shared.dtype)
        _check(gate, "gate", torch.float32, contiguous=False)
        if gate.dim() != 1 or gate.shape[0] != N:
            raise ValueError("gate must be one float per token")
        gs = gate.stride(0) if N > 1 else 1
    _call("ms_moe_combine", part.data_ptr(), ids.data_ptr(), _ptr(weights), h.data_ptr(), hs, _ptr(shared), scode,
          _ptr(gate), gs, out.data_ptr(), N, top, n_experts, H, _code(h.dtype), _stream())
    return out


# ------------------------------------------------------------------------------------------------ layer norm, side input
def layer_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out: Optional[torch.Tensor],
               delta: Optional[torch.Tensor] = None, delta_scale: Optional[torch.Tensor] = None,
               rows: Optional[torch.Tensor] = None, write_back: bool = True, bias: Optional[torch.Tensor] = None):
    """out[r] = weight * (v - mean v) / sqrt(mean (v - mean v)^2 + eps) (+ bias) with v = x[rows[r]] (+ delta_scale o delta[rows[r]]).
    x float32 [N, H] is the residual stream; with ``delta`` [N, H] the sum is written back to x (unless ``write_back`` is
    False).  ``weight`` None: only the sum, and ``out`` (if given) takes the summed rows rounded to its type.  ``out`` may
    be x itself (float): the rows are normed in place."""
    _check(x, "x", torch.float32)
    N, H = x.shape
    n_rows = N
    if rows is not None:
        _check(rows, "rows", torch.int32)
        n_rows = rows.numel()
    if weight is not None:
        _check(weight, "weight", torch.float32, (H,))
    if bias is not None:
        if weight is None:
            raise ValueError("a bias without a weight")
        _check(bias, "bias", torch.float32, (H,))
    if weight is not None or out is not None:
        _check(out, "out", None, (n_rows, H))
    dcode = 0
    if delta is not None:
        _check(delta, "delta", None, (N, H))
        dcode = _code(delta.dtype)
        if delta_scale is not None:
            _check(delta_scale, "delta_scale", torch.float32, (H,))
    elif delta_scale is not None:
        raise ValueError("a scale without an addend")
    _call("ms_layer_norm", x.data_ptr(), _ptr(delta), dcode, _ptr(delta_scale), _ptr(weight), _ptr(bias), _ptr(rows),
          _ptr(out), n_rows, H, float(eps), int(write_back), _code(out.dtype) if out is not None else F32, _stream())
    return out


def side_gate(z: torch.Tensor, token_ids: torch.Tensor, table: torch.Tensor, part: int, out: torch.Tensor) -> torch.Tensor:
    """out[n, j] = gelu_tanh(z[n, j]) * table[token_ids[n], part d + j] for z [N, d] (rows may be slices); table [V, parts d]."""
    N, d = z.shape
    zs = _rows2d(z, "z", table.dtype)
    _check(table, "table")
    if table.dim() != 2 or (part + 1) * d > table.shape[1] or part < 0:
        raise ValueError(f"part {part} of {d} entries is not within the table's rows of {table.shape[1]}")
    _check(token_ids, "token_ids", torch.int32, (N,))
    _check(out, "out", table.dtype, (N, d))
    _call("ms_side_gate", z.data_ptr(), zs, token_ids.data_ptr(), table.data_ptr(), table.shape[1], int(part), out.data_ptr(),
          N, d, _code(table.dtype), _stream())
    return out


# ------------------------------------------------------------------------------------------------ minGRU
def mingru_scan(zxg: torch.Tensor, bias_z: Optional[torch.Tensor], bias_x: Optional[torch.Tensor], state: torch.Tensor,
                ctx, out: torch.Tensor) -> torch.Tensor:
    """The minGRU recurrence over the step's portions, from and into ``state`` float [slots, C]: with the thirds pz | px | pg
    of a row of zxg [N, 3C]: z = sigmoid(pz + bias_z); u = px + bias_x; c = u + 1/2 (u >= 0) or sigmoid(u);
    S <- (1 - z) S + z c; out = S * silu(pg).  ``ctx.max_q_len`` bounds the portions' lengths."""
    C = state.shape[1]
    stride = _rows2d(zxg, "zxg", None, 3 * C)
    N = zxg.shape[0]
    os_ = _rows2d(out, "out", zxg.dtype, C)
    if out.shape[0] != N:
        raise ValueError("out has one row per token")
    for b, name in ((bias_z, "bias_z"), (bias_x, "bias_x")):
        if b is not None:
            _check(b, name, torch.float32, (C,))
    _check(state, "state", torch.float32, (None, C))
    R = ctx.num_requests
    _check(ctx.q_start, "q_start", torch.int32, (R + 1,))
    _check(ctx.state_slots, "state_slots", torch.int32, (R,))
    longest = max(1, int(ctx.max_q_len))
    chunk = int(_get("ms_mingru_chunk")())
    scratch = None
    if longest > chunk:      # a long portion's chunks are spread over blocks; their pairs and starting states pass through here
        scratch = torch.empty((R * (-(-longest // chunk)) * 2 + R) * C, dtype=torch.float32, device=zxg.device)
    _call("ms_mingru_scan", zxg.data_ptr(), stride, _ptr(bias_z), _ptr(bias_x), state.data_ptr(), ctx.q_start.data_ptr(),
          ctx.state_slots.data_ptr(), out.data_ptr(), os_, R, C, longest, _ptr(scratch), _code(zxg.dtype), _stream())
    return out


# ------------------------------------------------------------------------------------------------ window + pooled blocks
def _token_pages(kv, names=("k", "v")):
    """(key pages [P, heads, page, d], value pages, value size, whether the value pages are [P, heads, dv, page])."""
    k, v = kv.pages[names[0]], kv.pages[names[1]]
    if kv.transposed.get(names[0]):
        raise ValueError("these kernels read key pages as [page, head, slot, width]")
    flipped = bool(kv.transposed.get(names[1]))
    _check(k, "k pages")
    P, nkv, page, _ = k.shape
    _check(v, "v pages", k.dtype, (P, nkv, None, page) if flipped else (P, nkv, page, None))
    return k, v, (v.shape[2] if flipped else v.shape[3]), flipped


def pairs_rotate_store(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                       rot_dims: int, positions: torch.Tensor, inv_freq: torch.Tensor, inv_freq_v: torch.Tensor,
                       kv) -> torch.Tensor:
    """Rows of the packed projection [N, nh d + nkv d + nkv dv]: q and k heads turn over their first ``rot_dims`` entries
    (entries 2m, 2m + 1 by positions[n] * inv_freq[m]), value heads over all their entries (by positions[n] *
    inv_freq_v[m]); q in place, k and v into ``kv``'s pages at the tokens' slots (``kv`` None or not storing: q only)."""
    N = qkv.shape[0]
    width = (num_heads + num_kv_heads) * head_dim + num_kv_heads * value_dim
    stride = _rows2d(qkv, "qkv", None, width)
    _check(positions, "positions", torch.int32, (N,))
    _check(inv_freq, "inv_freq", torch.float32, (rot_dims // 2,))
    _check(inv_freq_v, "inv_freq_v", torch.float32, (value_dim // 2,))
    store = kv is not None and kv.store
    k = v = None
    page_size = 1
    flipped = False
    if store:
        k, v, dv, flipped = _token_pages(kv)
        _check(k, "k pages", qkv.dtype, (None, num_kv_heads, None, head_dim))
        if dv != value_dim:
            raise ValueError(f"the value pages hold values of {dv} entries, not {value_dim}")
        _check(kv.slot_mapping, "slot_mapping", torch.int32, (N,))
        page_size = k.shape[2]
    _call("ms_pairs_rotate_store", qkv.data_ptr(), stride, positions.data_ptr(), inv_freq.data_ptr(), inv_freq_v.data_ptr(),
          kv.slot_mapping.data_ptr() if store else None, _ptr(k), _ptr(v), N, num_heads, num_kv_heads, head_dim, value_dim,
          rot_dims, page_size, int(flipped), _code(qkv.dtype), _stream())
    return qkv


def pool_store(kv, pooled, ctx, pool: int) -> None:
    """For every token of the step that ends a block of ``pool`` tokens (its slot in ``pooled`` is not negative): the means
    of the block's keys and values, read back from ``kv``'s pages, go into ``pooled``'s pages "k" and "v"."""
    k, v, dv, flipped = _token_pages(kv)
    pk, pv, pdv, pflipped = _token_pages(pooled)
    P, nkv, page_size, d = k.shape
    _check(pk, "pooled k", k.dtype, (None, nkv, page_size, d))
    if pdv != dv or pflipped != flipped:
        raise ValueError("the pooled value pages must have the size and the layout of the tokens' value pages")
    N = ctx.num_tokens
    _check(pooled.slot_mapping, "pooled slots", torch.int32, (N,))
    _check(kv.block_table, "block_table", torch.int32)
    _call("ms_pool_store", k.data_ptr(), v.data_ptr(), kv.block_table.data_ptr(), kv.block_table.shape[1],
          _ptr(kv.table_rows), ctx.token_req.data_ptr(), ctx.positions.data_ptr(), pooled.slot_mapping.data_ptr(),
          pk.data_ptr(), pv.data_ptr(), N, nkv, d, dv, page_size, int(pool), int(flipped), _code(k.dtype), _stream())


def pooled_attention(q: torch.Tensor, kv, pooled, ctx, out: torch.Tensor, num_heads: int, scale: float, size: int,
                     pool: int, inv_freq_v: Optional[torch.Tensor] = None, turn_back: Optional[torch.Tensor] = None,
                     matrix_cores: Optional[bool] = None) -> torch.Tensor:
    """out[n, h] = softmax over the last ``size`` tokens up to n's position and over the pooled entry of every block of
    ``pool`` tokens that lies wholly before that window (block b: b pool + pool - 1 <= position - size), one softmax for
    both; tokens from ``kv``'s pages, block b from entry b of ``pooled``'s (None: no blocks).  With ``inv_freq_v`` the
    output's entries 2m, 2m + 1 are turned by -position * inv_freq_v[m].  q [N, >= nh d] row slices; out [N, nh dv].
    bfloat16 with transposed value pages, keys and values of one size that the matrix-core kernel has and pooled blocks
    goes there (``matrix_cores``: None decides by that, True insists, False keeps to the vector ALUs); it takes the cosines
    and sines of the angles from ``turn_back`` (``rope_table(positions, inv_freq_v)``), made here if not given."""
    k, v, dv, flipped = _token_pages(kv)
    P, nkv, page_size, d = k.shape
    _check(q, "q", k.dtype, contiguous=False)
    N = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < num_heads * d:
        raise ValueError(f"q must be [N, >= {num_heads * d}] with unit stride along rows, got {list(q.shape)}")
    _check(out, "out", k.dtype, (N, num_heads * dv))
    if num_heads % nkv:
        raise ValueError(f"{num_heads} query heads cannot share {nkv} key/value heads")
    pk = pv = ptab = None
    if pooled is not None and pool > 0:
        pk, pv, pdv, pflipped = _token_pages(pooled)
        _check(pk, "pooled k", k.dtype, (None, nkv, page_size, d))
        if pdv != dv or pflipped != flipped:
            raise ValueError("the pooled value pages must have the size and the layout of the tokens' value pages")
        ptab = pooled.block_table
        _check(ptab, "pooled table", torch.int32, tuple(kv.block_table.shape))
    else:
        pool = 0
    if inv_freq_v is not None:
        _check(inv_freq_v, "inv_freq_v", torch.float32, (dv // 2,))
    _check(ctx.token_req, "token_req", torch.int32, (N,))
    _check(ctx.positions, "positions", torch.int32, (N,))
    can = (q.dtype == torch.bfloat16 and flipped and dv == d and pool > 0 and scale > 0 and attention_mfma_supported(d, page_size)
           and q.data_ptr() % 16 == 0 and (N == 1 or q.stride(0) % 8 == 0))
    if matrix_cores and not can:
        raise UnsupportedShape("the matrix-core kernel takes bfloat16, transposed value pages of the keys' size (32, 64 or "
                               "128) and pages of a multiple of 16 tokens")
    if can and matrix_cores is not False:
        R = ctx.num_requests
        _check(ctx.q_start, "q_start", torch.int32, (R + 1,))
        _check(ctx.context_lens, "context_lens", torch.int32, (R,))
        if inv_freq_v is not None and turn_back is None:
            turn_back = rope_table(ctx.positions, inv_freq_v)
        if turn_back is not None:
            _check(turn_back, "turn_back", torch.float32, (N, d // 2, 2))
        try:
            _call("ms_pooled_attention_mfma", q.data_ptr(), q.stride(0) if N > 1 else q.shape[1], k.data_ptr(), v.data_ptr(),
                  kv.block_table.data_ptr(), pk.data_ptr(), pv.data_ptr(), ptab.data_ptr(), kv.block_table.shape[1],
                  _ptr(kv.table_rows), ctx.q_start.data_ptr(), ctx.context_lens.data_ptr(), _ptr(turn_back), out.data_ptr(),
                  num_heads * dv, R, N, max(1, ctx.max_q_len), num_heads, nkv, d, page_size, float(scale), int(size),
                  int(pool), _stream())
            return out
        except UnsupportedShape:        # more tiles than a launch holds: the vector-ALU kernel takes any step
            if matrix_cores:
                raise
    _call("ms_pooled_attention", q.data_ptr(), q.stride(0) if N > 1 else q.shape[1], k.data_ptr(), v.data_ptr(),
          kv.block_table.data_ptr(), _ptr(pk), _ptr(pv), _ptr(ptab), kv.block_table.shape[1], _ptr(kv.table_rows),
          _ptr(ctx.n_live_tokens), ctx.token_req.data_ptr(), ctx.positions.data_ptr(), _ptr(inv_freq_v), out.data_ptr(),
          num_heads * dv, N, num_heads, nkv, d, dv, page_size, float(scale), int(size), int(pool), int(flipped),
          _code(q.dtype), _stream())
    return out


# ------------------------------------------------------------------------------------------------ gated activations
def clamped_glu(gu: torch.Tensor, out: torch.Tensor, limit: float, alpha: float = 1.702) -> torch.Tensor:
    """gu [N, 2F] with gate and up interleaved: g = min(g, limit), u = clamp(u, -limit, limit),
    out = g * sigmoid(alpha g) * (u + 1), [N, F]."""
    F = gu.shape[1] // 2
    s_in = _rows2d(gu, "gu", None, 2 * F)
    s_out = _rows2d(out, "out", gu.dtype, F)
    if out.shape[0] != gu.shape[0]:
        raise ValueError("out has one row per row of gu")
    _call("ms_clamped_glu", gu.data_ptr(), s_in, out.data_ptr(), s_out, gu.shape[0], F, float(limit), float(alpha),
          _code(gu.dtype), _stream())
    return out


def gelu_tanh_glu(gu: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[n, f] = gelu_tanh(g) * u for gu [N, 2F] with gate and up interleaved (g0, u0, g1, u1, ...), the tanh form of the
    gelu: z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))."""
    N = gu.shape[0]
    F = gu.shape[1] // 2
    gs = _rows2d(gu, "gu", None, 2 * F)
    os_ = _rows2d(out, "out", gu.dtype, F)
    if out.shape[0] != N:
        raise ValueError("out must have a row per row of gu")
    _call("ms_gelu_tanh_glu", gu.data_ptr(), gs, out.data_ptr(), os_, N, F, _code(gu.dtype), _stream())
    return out


def scaled_swiglu(gu: torch.Tensor, out: torch.Tensor, factor: Optional[torch.Tensor] = None,
                  row_item: Optional[torch.Tensor] = None) -> torch.Tensor:
    """gu [rows, 2F] with gate and up interleaved: out = silu(s g) * (s u) with s = factor[row_item[p]] for row p
    (factor[p] without ``row_item``; 1 without ``factor``); rows with a negative ``row_item`` are left alone."""
    F = gu.shape[1] // 2
    s_in = _rows2d(gu, "gu", None, 2 * F)
    s_out = _rows2d(out, "out", gu.dtype, F)
    n = gu.shape[0]
    if out.shape[0] != n:
        raise ValueError("out has one row per row of gu")
    if factor is not None:
        _check(factor, "factor", torch.float32)
    if row_item is not None:
        _check(row_item, "row_item", torch.int32)
        if row_item.numel() < n:
            raise ValueError("row_item names an item for every row")
    _call("ms_scaled_swiglu", gu.data_ptr(), s_in, _ptr(factor), _ptr(row_item), out.data_ptr(), s_out, n, F,
          _code(gu.dtype), _stream())
    return out
