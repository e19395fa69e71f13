"""Python face of the HIP kernels: checks operands against what a kernel and
its grid assume, then launches it on the current stream.  Every function here
runs hand-written device code; none has a host or library stand-in.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..cache.layout import k_page_shape, v_page_shape
from ..errors import KernelError, Unsupported
from . import lib as _lib

PAGE_TOKENS = 64

_VOID = ctypes.c_void_p
_INT = ctypes.c_int
_FLT = ctypes.c_float
_SIZE = ctypes.c_size_t
_U64 = ctypes.c_uint64
_I64 = ctypes.c_longlong

_CORE_SIGNATURES = {
    "nnis_embed": [_VOID, _VOID, _INT, _VOID, _INT, _INT, _INT, _FLT, _VOID],
    "nnis_embed_packed": [_VOID, _VOID, _VOID, _INT, _INT, _INT, _FLT, _VOID],
    "nnis_step_tables": [_VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _VOID, _INT, _VOID, _VOID, _VOID, _VOID, _VOID],
    "nnis_rmsnorm": [_VOID, _INT, _VOID, _INT, _VOID, _INT, _VOID, _INT, _VOID, _INT, _INT, _FLT, _VOID],
    "nnis_rope_kv_write": [_VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _INT,
                           _VOID, _INT, _INT, _INT, _INT, _INT, _VOID],
    "nnis_rope_kv_write_wide": [_VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _INT,
                                _VOID, _INT, _INT, _INT, _INT, _INT, _INT, _VOID, _INT, _VOID],
    "nnis_rope_kv_write_shared": [_VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _INT,
                                  _VOID, _INT, _INT, _INT, _INT, _INT, _INT, _VOID, _INT, _INT, _VOID],
    "nnis_branch_sum": [_VOID, _VOID, _INT, _INT, _I64, _VOID, _INT, _VOID],
    "nnis_scale_rows": [_VOID, _FLT, _I64, _VOID],
    "nnis_silu_mul": [_VOID, _INT, _VOID, _INT, _INT, _INT, _VOID],
    "nnis_embed_pair": [_VOID, _VOID, _VOID, _INT, _VOID, _INT, _INT, _VOID, _INT, _INT, _I64, _I64, _VOID, _VOID, _INT, _INT, _VOID],
    "nnis_stream_step": [_VOID, _INT, _INT, _INT, _VOID, _INT, _VOID, _VOID, _VOID, _VOID, _VOID, _INT, _INT, _FLT, _VOID, _INT,
                         _VOID, _INT, _VOID],
    "nnis_branch_mean": [_VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _FLT, _VOID, _INT, _VOID],
    "nnis_gated_act": [_VOID, _INT, _VOID, _INT, _INT, _INT, _INT, _VOID],
    "nnis_add_bias": [_VOID, _INT, _VOID, _INT, _INT, _INT, _VOID],
    "nnis_tanh_norm_step": [_VOID, _VOID, _VOID, _INT, _VOID, _VOID, _FLT, _VOID, _VOID, _VOID, _VOID, _FLT, _INT, _VOID, _INT, _VOID,
                            _INT, _INT, _VOID],
    "nnis_tanh_cap": [_VOID, _FLT, _I64, _VOID],
    "nnis_argmax": [_VOID, _VOID, _INT, _INT, _VOID, _VOID],
    "nnis_argmax_scratch": [_INT, _INT],
    "nnis_argmax_static": [_VOID, _VOID, _INT, _INT, _VOID],
    "nnis_gemm_ordered": [_VOID, _INT, _VOID, _INT, _VOID, _INT, _INT, _INT, _INT, _VOID],
    "nnis_gemm_bf16": [_VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _VOID, _SIZE, _VOID],
    "nnis_gemm_fused": [_VOID, _VOID, _VOID, _VOID, _INT, _FLT, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _VOID, _INT,
                        _VOID, _VOID, _VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _VOID, _INT, _VOID],
    "nnis_gemm_residual_parts": [_INT, _INT],
    "nnis_gemm_tile": [_INT, _INT, _INT],
    "nnis_gemm_takes_pair": [_INT, _INT, _INT, _SIZE],
    "nnis_gemm_residual": [_VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _INT, _VOID, _SIZE, _VOID, _VOID],
    "nnis_gemm_residual_tanh": [_VOID, _VOID, _VOID, _VOID, _VOID, _FLT, _VOID, _VOID, _FLT, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT,
                                _VOID, _SIZE, _VOID, _VOID],
    "nnis_gemm_scaled": [_VOID, _VOID, _INT, _FLT, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _VOID, _INT, _VOID, _VOID,
                         _VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _VOID, _INT, _VOID, _SIZE, _VOID],
    "nnis_gemm_residual_runs_fits": [_INT, _INT, _INT, _INT, _INT],
    "nnis_gemm_residual_runs": [_VOID, _INT, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _VOID,
                                _VOID],
    "nnis_pack_weight": [_VOID, _VOID, _INT, _INT, _VOID],
    "nnis_sample": [_VOID, _VOID, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _VOID],
}
_ATTN_SIGNATURES = {
    "nnis_attention_rows": [_VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT,
                            _INT, _INT, _FLT, _INT, _FLT, _VOID],
    "nnis_attention_rows_more": [_VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT,
                                 _INT, _INT, _FLT, _INT, _FLT, _INT, _VOID, _INT, _VOID, _VOID],
    "nnis_attention_rows_pooled": [_VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT,
                                   _INT, _INT, _FLT, _INT, _FLT, _INT, _VOID, _INT, _VOID, _VOID, _VOID, _VOID, _INT, _INT, _VOID],
    "nnis_attention_prefill_bf16_pooled": [_VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _VOID, _VOID, _VOID, _INT,
                                           _INT, _INT, _INT, _FLT, _INT, _INT, _FLT, _INT, _VOID, _INT, _VOID,
                                           _VOID, _VOID, _VOID, _INT, _INT, _VOID],
    "nnis_attention_decode_bf16_pooled": [_VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _FLT,
                                          _INT, _INT, _VOID, _INT, _INT, _INT, _FLT, _INT, _VOID, _INT, _VOID,
                                          _VOID, _VOID, _VOID, _INT, _INT, _VOID],
    "nnis_attention_prefill_tile_rows": [_INT, _INT, _INT],
    "nnis_attention_prefill_bf16": [_VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _VOID, _VOID, _VOID, _INT,
                                    _INT, _INT, _INT, _FLT, _INT, _INT, _FLT, _VOID],
    "nnis_attention_prefill_bf16_more": [_VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _VOID, _VOID, _VOID, _INT,
                                         _INT, _INT, _INT, _FLT, _INT, _INT, _FLT, _INT, _VOID, _INT, _VOID, _VOID],
    "nnis_attention_decode_bf16_more": [_VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _FLT,
                                        _INT, _INT, _VOID, _INT, _INT, _INT, _FLT, _INT, _VOID, _INT, _VOID, _VOID],
    "nnis_attention_prefill_max_waves": [_INT, _INT, _INT],
    "nnis_attention_decode_bf16": [_VOID, _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _FLT,
                                   _INT, _INT, _VOID, _INT, _INT, _INT, _FLT, _VOID],
    "nnis_attention_combine": [_VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID],
    "nnis_attention_decode_max_waves": [_INT, _INT],
}

_RECURRENT_SIGNATURES = {
    "nnis_conv_silu": [_VOID, _INT, _INT, _VOID, _VOID, _INT, _VOID, _VOID, _VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _INT,
                       _INT, _VOID],
    "nnis_selective_scan": [_VOID, _INT, _VOID, _VOID, _VOID, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _VOID, _VOID, _INT, _INT, _INT,
                            _VOID, _INT, _INT, _INT, _VOID, _VOID, _VOID],
    "nnis_gla_scan": [_VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _FLT, _VOID, _VOID, _VOID, _INT, _INT, _INT, _INT,
                      _VOID, _INT, _INT, _VOID, _VOID, _VOID],
    "nnis_gla_scan_turned": [_VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _VOID, _VOID, _INT, _INT, _VOID, _FLT, _VOID,
                             _VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _INT, _INT, _VOID, _VOID, _VOID],
    "nnis_gated_delta": [_VOID, _INT, _INT, _VOID, _VOID, _VOID, _FLT, _FLT, _VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _INT, _VOID,
                         _VOID, _VOID],
    "nnis_gla_decays": [_VOID, _VOID, _INT, _INT, _FLT, _VOID],
    "nnis_head_norm_gate": [_VOID, _VOID, _INT, _INT, _VOID, _INT, _VOID, _INT, _INT, _INT, _INT, _FLT, _VOID],
    "nnis_min_gru": [_VOID, _INT, _INT, _VOID, _VOID, _INT, _VOID, _VOID, _VOID, _INT, _INT, _VOID, _INT, _INT, _INT, _VOID, _VOID, _VOID],
}

_SUBLAYER_SIGNATURES = {
    "nnis_cast_rows": [_VOID, _INT, _VOID, _INT, _VOID, _INT, _INT, _VOID],
    "nnis_rms_post_step": [_VOID, _VOID, _INT, _VOID, _INT, _FLT, _FLT, _VOID, _INT, _INT, _INT, _VOID, _VOID, _INT, _VOID],
    "nnis_rms_between": [_VOID, _VOID, _INT, _VOID, _VOID, _INT, _FLT, _VOID, _INT, _INT, _INT, _VOID, _VOID, _INT, _VOID],
    "nnis_route": [_VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _VOID, _VOID, _INT, _INT, _VOID],
    "nnis_poly_norm": [_VOID, _INT, _VOID, _FLT, _VOID, _INT, _INT, _INT, _VOID],
    "nnis_router_logits": [_VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _VOID],
    "nnis_route_top": [_VOID, _VOID, _INT, _INT, _INT, _INT, _VOID, _VOID, _INT, _INT, _VOID],
    "nnis_routed_act": [_VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _VOID],
    "nnis_rows_axpy": [_VOID, _INT, _VOID, _INT, _VOID, _INT, _INT, _VOID],
    "nnis_sigmoid_gate": [_VOID, _INT, _VOID, _INT, _INT, _INT, _INT, _VOID],
    "nnis_head_norm_write": [_VOID, _INT, _INT, _INT, _INT, _INT, _VOID, _INT, _VOID, _VOID, _INT, _FLT, _VOID, _VOID, _INT, _INT, _INT,
                             _VOID, _VOID, _VOID, _VOID, _INT, _VOID, _INT, _INT, _INT, _INT, _INT, _INT, _VOID],
    "nnis_pool_blocks": [_VOID, _VOID, _INT, _VOID, _INT, _VOID, _VOID, _VOID, _INT, _VOID, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _INT,
                         _VOID],
}

_LATENT_SIGNATURES = {
    "nnis_latent_prepare": [_VOID, _INT, _INT, _INT, _INT, _INT, _INT, _VOID, _VOID, _INT, _FLT, _VOID, _VOID, _INT, _VOID, _VOID, _VOID,
                            _INT, _VOID, _VOID, _INT, _VOID, _INT, _VOID, _VOID],
    "nnis_latent_rotate_q": [_VOID, _INT, _INT, _INT, _INT, _INT, _INT, _VOID, _VOID, _INT, _VOID, _VOID],
    "nnis_head_scale": [_VOID, _INT, _VOID, _INT, _INT, _INT, _VOID],
    "nnis_head_scale_of": [_VOID, _INT, _VOID, _INT, _INT, _INT, _INT, _VOID],
    "nnis_heads_linear": [_VOID, _INT, _VOID, _INT, _VOID, _VOID, _INT, _INT, _INT, _INT, _INT, _VOID],
}

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


def _pages_fit(k_pages: torch.Tensor, v_pages: torch.Tensor, kv_heads: int, head_dim: int, value_dim: Optional[int] = None) -> bool:
    """Key and value pages [pages, ...] in the cache's layout for these sizes, contiguous."""
    return (tuple(k_pages.shape[1:]) == k_page_shape(kv_heads, head_dim)
            and tuple(v_pages.shape[1:]) == v_page_shape(kv_heads, value_dim or head_dim)
            and k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.shape[0] == v_pages.shape[0])


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}") from None


def bind(module: str, signatures):
    """Loads a kernel module (one that ``kernels.lib`` has built in, or one that a part registered there with
    ``register_module``) and declares its entry points: ``signatures`` maps a name to its argument types; every
    entry point returns an int, 0 or an error whose text ``nnis_last_error()`` holds (``check`` raises it)."""
    return _bind(module, signatures)


def stream() -> int:
    """The raw handle of the stream that launches go to (the last argument of every entry point)."""
    return _stream()


def check(lib, status: int) -> None:
    _check(lib, status)


def _bind(module: str, signatures):
    lib = _lib.load_module(module)
    if not getattr(lib, "_nnis_bound", False):
        for name, argtypes in signatures.items():
            fn = getattr(lib, name, None)
            if fn is None:
                continue  # a kernel that is not in this build; calling it raises below
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        lib._nnis_bound = True
    return lib


_core = None
_attn = {}
_recurrent = None


def recurrent():
    """The module of the mixers that carry state (convolution, selective scan, gated linear attention)."""
    global _recurrent
    if _recurrent is None:
        _recurrent = _bind("recurrent", _RECURRENT_SIGNATURES)
    return _recurrent


_latent = None


def latent():
    """The module of attention over a cached latent (norms of the latents, rotation, cache write, gates)."""
    global _latent
    if _latent is None:
        _latent = _bind("latent", _LATENT_SIGNATURES)
    return _latent


_sublayer = None


def sublayer():
    """The module of what lies between the projections of sublayers that norm their outputs, gate or pool their
    heads, or route their tokens."""
    global _sublayer
    if _sublayer is None:
        _sublayer = _bind("sublayer", _SUBLAYER_SIGNATURES)
    return _sublayer


def core():
    global _core
    if _core is None:
        _core = _bind("core", _CORE_SIGNATURES)
    return _core


ATTENTION_MOST_CHANNELS = 256  # of the matrix-core kernels
ATTENTION_ROWS_MOST_CHANNELS = 1024  # of the 32-bit row kernel, which takes what the others do not (a lane's outputs then live in scratch memory)


_wide_heads = set()  # (key channels, value channels) beyond the matrix-core kernels' that a mixer has accepted the row kernel for


def attention_check(head_dim: int, value_dim: Optional[int] = None, most: int = ATTENTION_MOST_CHANNELS) -> None:
    """Raises ``Unsupported`` for a head size that the attention kernels do not take: up to ``most`` channels, by
    default what the matrix-core kernels carry.  A mixer that accepts the row kernel's pace for wider heads asks
    with ``ATTENTION_ROWS_MOST_CHANNELS``; only sizes accepted so are loaded beyond the default."""
    if head_dim <= 0 or head_dim > most:
        raise Unsupported(f"the attention kernels take a head_dim up to {most}, got {head_dim}")
    if value_dim is not None and value_dim != head_dim and not 0 < value_dim <= most:
        raise Unsupported(f"the attention kernels take values of up to {most} channels, got {value_dim}")
    if most > ATTENTION_MOST_CHANNELS:
        _wide_heads.add((head_dim, value_dim or head_dim))


def attention_module_name(head_dim: int, value_dim: Optional[int] = None, softcap: float = 0.0, extras=None, pooled=None) -> str:
    """The module compiled for keys of ``head_dim`` channels and values of ``value_dim`` (None: as the keys), with a
    cap of the scores (``softcap`` > 0) or without, with the scores' extras (``ScoreExtras``) or without, and, with the
    extras, with pooled blocks beside a window (``PooledBlocks``) or without."""
    wide = value_dim is not None and value_dim != head_dim
    return ((f"attn_hd{head_dim}v{value_dim}" if wide else f"attn_hd{head_dim}") + ("c" if softcap else "")
            + ("xp" if pooled is not None else ("x" if extras else "")))


def attention_module(head_dim: int, value_dim: Optional[int] = None, softcap: float = 0.0, extras=None, pooled=None):
    name = attention_module_name(head_dim, value_dim, softcap, extras, pooled)
    if name not in _attn:
        accepted = (head_dim, value_dim or head_dim) in _wide_heads
        attention_check(head_dim, value_dim, ATTENTION_ROWS_MOST_CHANNELS if accepted else ATTENTION_MOST_CHANNELS)
        _attn[name] = _bind(name, _ATTN_SIGNATURES)
    return _attn[name]


def _check(lib, status: int) -> None:
    if status != 0:
        raise KernelError(lib.nnis_last_error().decode(errors="replace"))


_device_index: Optional[int] = None


def bind_device(index: int) -> None:
    """Names the one GPU whose streams this process's launches go to.  The
    runtime calls it when it is made (and makes that device current); a
    second runtime on another GPU is refused, because every launch below
    takes the bound device's current stream and the per-device arrays
    (``argmax_no_alloc``, the products' workspace) are looked up for it."""
    global _device_index
    if _device_index is not None and _device_index != int(index):
        raise KernelError(f"this process already runs its kernels on cuda:{_device_index}; a process drives one GPU "
                          f"(cuda:{int(index)} was asked for)")
    _device_index = int(index)


def bound_device() -> Optional[int]:
    return _device_index


def _stream() -> int:
    """The bound device's current stream (a raw handle:
    ``torch.cuda.current_stream().cuda_stream`` builds a Python stream object
    on every call, which cost a third of an operation's time on the host)."""
    if _device_index is None:
        bind_device(torch.cuda.current_device())  # kernels called without a runtime (tests of one kernel)
    return torch._C._cuda_getCurrentRawStream(_device_index)


def _dev(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise KernelError(f"{what} must live on the GPU; this library has no host path")
    if not t.is_contiguous():
        raise KernelError(f"{what} must be contiguous")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# ---------------------------------------------------------------------------

def embed(ids: torch.Tensor, table, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] widened to 32-bit, times ``scale``; ids outside the table give a zero row.
    ``table``: a matrix [vocab, width], or the ``PackedWeight`` of one (a table that a head shares)."""
    _dev(ids, "ids"), _dev(table, "embedding table"), _dev(out, "out")
    tokens, width = out.shape
    if ids.dtype != torch.int32 or ids.numel() < tokens:
        raise KernelError(f"embed: ids must be int32 with at least {tokens} entries")
    if isinstance(table, PackedWeight):
        if table.shape[1] != width or out.dtype != torch.float32:
            raise KernelError(f"embed: packed table {table.shape} / out {tuple(out.shape)} {out.dtype} do not fit")
        lib = core()
        _check(lib, lib.nnis_embed_packed(ids.data_ptr(), table.data_ptr(), out.data_ptr(), tokens, width, table.shape[0], float(scale), _stream()))
        return out
    if table.dim() != 2 or table.shape[1] != width or out.dtype != torch.float32:
        raise KernelError(f"embed: table {tuple(table.shape)} / out {tuple(out.shape)} {out.dtype} do not fit")
    lib = core()
    _check(lib, lib.nnis_embed(ids.data_ptr(), table.data_ptr(), _code(table), out.data_ptr(), tokens, width,
                               table.shape[0], float(scale), _stream()))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = rmsnorm(x [+ delta]) * weight.  Without ``rows`` and with ``delta``
    the sum is written back into ``x`` (32-bit).  With ``rows`` (int32), output
    row r reads input row rows[r]."""
    _dev(x, "x"), _dev(weight, "norm weight"), _dev(out, "out")
    width = x.shape[-1]
    if weight.numel() != width or out.shape[-1] != width:
        raise KernelError(f"rmsnorm: width {width} against weight {tuple(weight.shape)} and out {tuple(out.shape)}")
    out_rows = out.numel() // width
    if rows is None:
        if x.numel() // width != out_rows:
            raise KernelError(f"rmsnorm: {x.numel() // width} input rows against {out_rows} output rows")
    else:
        _dev(rows, "rows")
        if rows.dtype != torch.int32 or rows.numel() < out_rows:
            raise KernelError("rmsnorm: rows must be int32 with one entry per output row")
    if delta is not None:
        _dev(delta, "delta")
        if delta.shape != x.shape:
            raise KernelError(f"rmsnorm: delta {tuple(delta.shape)} against x {tuple(x.shape)}")
    lib = core()
    _check(lib, lib.nnis_rmsnorm(x.data_ptr(), _code(x), _ptr(delta), _code(delta) if delta is not None else 0,
                                 weight.data_ptr(), _code(weight), out.data_ptr(), _code(out), _ptr(rows), out_rows,
                                 width, float(eps), _stream()))
    return out


def rope_kv_write(qkv: torch.Tensor, q_out: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                  rot_dim: int, tok_slot: torch.Tensor, tok_pos: torch.Tensor, k_pages: Optional[torch.Tensor],
                  v_pages: Optional[torch.Tensor], block_table: Optional[torch.Tensor], heads: int, kv_heads: int,
                  head_dim: int, value_dim: Optional[int] = None, bias: Optional[torch.Tensor] = None,
                  values_from_keys: bool = False) -> torch.Tensor:
    """``values_from_keys``: the rows hold queries and keys only, and a head's
    value is its key as projected, before the rotation.
    Rotates queries and keys by their positions and writes keys and values
    into the pages of each token's slot.  ``k_pages`` and ``v_pages`` are
    ``[pages, *k_page_shape(kv_heads, head_dim)]`` and ``[pages,
    *v_page_shape(kv_heads, value_dim)]`` (``cache/layout.py``); both ``None``
    for a run that keeps no cache of its own.  ``value_dim``: channels of a
    value head (None: as the keys).  ``bias``: one entry per column of
    ``qkv``, added before the rotation."""
    _dev(qkv, "qkv"), _dev(q_out, "q_out"), _dev(tok_slot, "tok_slot"), _dev(tok_pos, "tok_pos")
    tokens = qkv.shape[0]
    value_dim = value_dim or head_dim
    if values_from_keys and value_dim != head_dim:
        raise KernelError(f"rope_kv_write: values that are the keys have their size ({head_dim}), not {value_dim}")
    if qkv.shape[1] != (heads + kv_heads) * head_dim + (0 if values_from_keys else kv_heads * value_dim) or q_out.shape != (tokens, heads * head_dim):
        raise KernelError(f"rope_kv_write: qkv {tuple(qkv.shape)} / q_out {tuple(q_out.shape)} do not fit "
                          f"{heads}+{kv_heads} heads of {head_dim} and {kv_heads} of {value_dim}")
    if bias is not None:
        _dev(bias, "bias")
        if bias.numel() != qkv.shape[1]:
            raise KernelError(f"rope_kv_write: a bias of {bias.numel()} entries for rows of {qkv.shape[1]}")
    if tok_slot.dtype != torch.int32 or tok_pos.dtype != torch.int32 or tok_slot.numel() < tokens or tok_pos.numel() < tokens:
        raise KernelError("rope_kv_write: tok_slot / tok_pos must be int32 with one entry per token")
    table_positions = 0
    if cos is not None:
        _dev(cos, "cos"), _dev(sin, "sin")
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[1] != rot_dim // 2:
            raise KernelError(f"rope_kv_write: tables {tuple(cos.shape)} do not fit rot_dim {rot_dim} in float32")
        table_positions = cos.shape[0]
    max_pages = 0
    cache_code = 0
    if k_pages is not None:
        _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(block_table, "block_table")
        if not _pages_fit(k_pages, v_pages, kv_heads, head_dim, value_dim):
            raise KernelError(f"rope_kv_write: page shapes {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not fit")
        if block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise KernelError("rope_kv_write: block_table must be int32 [slots, pages]")
        max_pages = block_table.shape[1]
        cache_code = _code(k_pages)
    lib = core()
    _check(lib, lib.nnis_rope_kv_write_shared(qkv.data_ptr(), _code(qkv), q_out.data_ptr(), _code(q_out), _ptr(cos), _ptr(sin),
                                              table_positions, rot_dim, tok_slot.data_ptr(), tok_pos.data_ptr(),
                                              _ptr(k_pages), _ptr(v_pages), cache_code, _ptr(block_table), max_pages, tokens,
                                              heads, kv_heads, head_dim, value_dim, _ptr(bias),
                                              _code(bias) if bias is not None else 0, 1 if values_from_keys else 0, _stream()))
    return q_out


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(gate_up, "gate_up"), _dev(out, "out")
    tokens, inner = out.shape
    if gate_up.shape != (tokens, 2 * inner):
        raise KernelError(f"silu_mul: gate_up {tuple(gate_up.shape)} against out {tuple(out.shape)}")
    lib = core()
    _check(lib, lib.nnis_silu_mul(gate_up.data_ptr(), _code(gate_up), out.data_ptr(), _code(out), tokens, inner, _stream()))
    return out


STATIC_SCRATCH_WORDS = 65536  # NNIS_STATIC_SCRATCH_WORDS of csrc/nnis_noalloc.h


def argmax(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(logits, "logits"), _dev(out, "out")
    rows, vocab = logits.shape
    if logits.dtype != torch.float32 or out.dtype != torch.int32 or out.numel() < rows:
        raise KernelError("argmax: logits must be float32 [rows, vocab] and out int32 [rows]")
    if not logits.is_contiguous():
        raise KernelError("argmax: logits must be contiguous")
    lib = core()
    need = lib.nnis_argmax_scratch(rows, vocab)
    if need <= STATIC_SCRATCH_WORDS:
        # the array that the library holds on the GPU: nothing to allocate (calls follow one another on one stream)
        _check(lib, lib.nnis_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, _stream()))
        return out
    scratch = torch.empty(max(1, need), dtype=torch.float32, device=logits.device)
    _check(lib, lib.nnis_argmax(logits.data_ptr(), out.data_ptr(), rows, vocab, scratch.data_ptr(), _stream()))
    return out


def argmax_no_alloc(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``argmax`` for callers that cannot allocate: the first pass's results go
    through a fixed array that the library holds on the GPU (256 KB; enough
    for 2 * rows * ceil(vocab / 4096) <= 65,536 words, beyond that the call
    is refused).  Calls on one GPU share the array: keep them in order on one
    stream."""
    _dev(logits, "logits"), _dev(out, "out")
    rows, vocab = logits.shape
    if logits.dtype != torch.float32 or out.dtype != torch.int32 or out.numel() < rows:
        raise KernelError("argmax: logits must be float32 [rows, vocab] and out int32 [rows]")
    lib = core()
    _check(lib, lib.nnis_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, _stream()))
    return out


def gemm_ordered(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = x[M, K] @ w[N, K]^T, each element one ascending-k chain of
    32-bit fused multiply-adds."""
    _dev(x, "x"), _dev(w, "weight"), _dev(out, "out")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or out.shape != (m, n):
        raise KernelError(f"gemm: x {tuple(x.shape)} w {tuple(w.shape)} out {tuple(out.shape)} do not fit")
    lib = core()
    _check(lib, lib.nnis_gemm_ordered(x.data_ptr(), _code(x), w.data_ptr(), _code(w), out.data_ptr(), _code(out), m, n, k,
                                      _stream()))
    return out


class StepTables:
    """What a step's kernels would look up through each token's slot and
    position, gathered once by token (``step_tables``): ``cos`` / ``sin``
    float32 [tokens, rot_dim / 2], each token's rows of the rotation tables;
    ``page`` int32 [tokens], the cache page of each token's position (-1 for a
    padding row); ``pages`` int32 [tokens, pages a slot may hold], for a step
    of single tokens the pages of each token's sequence up to its position.
    Any of them is None where it was not asked for."""

    def __init__(self, tokens, cos=None, sin=None, page=None, pages=None):
        self.tokens, self.cos, self.sin, self.page, self.pages = tokens, cos, sin, page, pages


def step_tables(tok_slot: torch.Tensor, tok_pos: torch.Tensor, tokens: int, cos: Optional[torch.Tensor] = None,
                sin: Optional[torch.Tensor] = None, block_table: Optional[torch.Tensor] = None,
                sequence_pages: bool = False) -> StepTables:
    """One kernel at the start of a step; see ``StepTables``.  ``cos`` / ``sin``:
    rotation tables [positions, half]; ``block_table``: int32 [slots, pages];
    ``sequence_pages``: also each token's sequence's pages (a decode step).
    The positions live on the device, where nothing can refuse them: the
    caller sees to it that every position is below ``cos.shape[0]`` and
    below ``block_table.shape[1] * 64`` (the engine refuses a step beyond the
    model's positions before it launches anything, and its tables reach that
    far); the kernel's clamps of a position beyond either are a guard against
    reading out of bounds, not a result."""
    _dev(tok_slot, "tok_slot"), _dev(tok_pos, "tok_pos")
    if tok_slot.dtype != torch.int32 or tok_pos.dtype != torch.int32 or min(tok_slot.numel(), tok_pos.numel()) < tokens:
        raise KernelError("step_tables: tok_slot / tok_pos must be int32 with one entry per token")
    out = StepTables(tokens)
    half = positions = max_pages = 0
    if cos is not None:
        _dev(cos, "cos"), _dev(sin, "sin")
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2:
            raise KernelError("step_tables: rotation tables must be float32 [positions, half]")
        positions, half = cos.shape
        out.cos = torch.empty((tokens, half), dtype=torch.float32, device=cos.device)
        out.sin = torch.empty((tokens, half), dtype=torch.float32, device=cos.device)
    if block_table is not None:
        _dev(block_table, "block_table")
        if block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise KernelError("step_tables: block_table must be int32 [slots, pages]")
        max_pages = block_table.shape[1]
        out.page = torch.empty(tokens, dtype=torch.int32, device=block_table.device)
        if sequence_pages:
            out.pages = torch.empty((tokens, max_pages), dtype=torch.int32, device=block_table.device)
    lib = core()
    _check(lib, lib.nnis_step_tables(tok_slot.data_ptr(), tok_pos.data_ptr(), tokens, _ptr(cos), _ptr(sin), half, positions,
                                     _ptr(block_table), max_pages, _ptr(out.cos), _ptr(out.sin), _ptr(out.page),
                                     _ptr(out.pages), _stream()))
    return out


class ScoreExtras:
    """What an attention may do to its scores beyond scale and cap, each off
    when zero or None.  ``keep_first``: with a window, keys at positions below
    this stay visible to every later query.  ``bias``: float32 [heads, reach +
    1], added to the scaled score of a key ``n`` positions back from its
    query, row min(n, reach) (a table by distance, one column set per head).
    ``sink``: float32 [heads], a score that joins the softmax's denominator
    once and has no value (exp(sink) is added to the sum of the weights)."""

    def __init__(self, keep_first: int = 0, bias: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None):
        self.keep_first, self.bias, self.sink = int(keep_first), bias, sink
        self.reach = 0 if bias is None else bias.shape[1] - 1

    def __bool__(self) -> bool:
        return bool(self.keep_first) or self.bias is not None or self.sink is not None

    def check(self, heads: int) -> None:
        for t, what in ((self.bias, "bias"), (self.sink, "sink")):
            if t is not None:
                _dev(t, f"attention {what}")
                if t.dtype != torch.float32 or t.shape[0] != heads or t.dim() != (2 if what == "bias" else 1):
                    raise KernelError(f"attention: the {what} must be float32 with a row per head ({heads}), got {tuple(t.shape)} {t.dtype}")
        if self.keep_first < 0:
            raise KernelError(f"attention: keep_first must not be negative, got {self.keep_first}")


class PooledBlocks:
    """Beside a window of ``window`` tokens: pages whose entry b holds one key
    and one value for the tokens b * pool .. b * pool + pool - 1 of a
    sequence (their means), with a block table of their own.  A query at
    position p sees entry b once the whole block has left its window, b * pool
    + pool - 1 <= p - window, in the same softmax as the window's keys."""

    def __init__(self, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor, pool: int):
        self.k_pages, self.v_pages, self.block_table, self.pool = k_pages, v_pages, block_table, int(pool)

    def check(self, k_pages, v_pages, kv_heads: int, head_dim: int, value_dim: int, window: int) -> None:
        _dev(self.k_pages, "pooled k_pages"), _dev(self.v_pages, "pooled v_pages"), _dev(self.block_table, "pooled block_table")
        if self.pool <= 0 or not window:
            raise KernelError(f"attention: pooled blocks of {self.pool} tokens beside a window of {window}")
        if not _pages_fit(self.k_pages, self.v_pages, kv_heads, head_dim, value_dim) or self.k_pages.dtype != k_pages.dtype \
                or self.v_pages.dtype != v_pages.dtype:
            raise KernelError(f"attention: pooled page shapes {tuple(self.k_pages.shape)} / {tuple(self.v_pages.shape)} do not fit the keys'")
        if self.block_table.dtype != torch.int32 or self.block_table.dim() != 2:
            raise KernelError("attention: the pooled block_table must be int32 [slots, pages]")


def attention_rows(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                   block_table: torch.Tensor, tok_slot: torch.Tensor, tok_pos: torch.Tensor, heads: int, kv_heads: int,
                   head_dim: int, scale: float, window: int = 0, value_dim: Optional[int] = None,
                   softcap: float = 0.0, extras: Optional[ScoreExtras] = None, pooled: Optional["PooledBlocks"] = None) -> torch.Tensor:
    """Causal attention of each token over the cached keys of its slot up to
    its own position (32-bit arithmetic, any storage type).  ``value_dim``:
    channels of a value head and of a head's output (None: as the keys).
    ``softcap`` > 0: a score s counts as softcap * tanh(s / softcap).
    ``pooled``: beside a window, one key and value for every block of tokens
    that lies wholly before it (``PooledBlocks``), in the same softmax."""
    _dev(q, "q"), _dev(out, "out"), _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(block_table, "block_table")
    tokens = q.shape[0]
    value_dim = value_dim or head_dim
    if q.shape != (tokens, heads * head_dim) or out.shape != (tokens, heads * value_dim):
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {heads} heads of {head_dim} "
                          f"with values of {value_dim}")
    if not _pages_fit(k_pages, v_pages, kv_heads, head_dim, value_dim):
        raise KernelError(f"attention: page shapes {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not fit")
    if k_pages.dtype != v_pages.dtype:
        raise KernelError("attention: key and value pages differ in type")
    if tok_slot.dtype != torch.int32 or tok_pos.dtype != torch.int32 or block_table.dtype != torch.int32:
        raise KernelError("attention: tok_slot, tok_pos and block_table must be int32")
    lib = attention_module(head_dim, value_dim, softcap, extras, pooled)
    if pooled is not None:
        extras = extras or ScoreExtras()
        extras.check(heads)
        pooled.check(k_pages, v_pages, kv_heads, head_dim, value_dim, window)
        _check(lib, lib.nnis_attention_rows_pooled(q.data_ptr(), _code(q), out.data_ptr(), _code(out), k_pages.data_ptr(),
                                                   v_pages.data_ptr(), _code(k_pages), block_table.data_ptr(), block_table.shape[1],
                                                   tok_slot.data_ptr(), tok_pos.data_ptr(), tokens, heads, kv_heads, head_dim,
                                                   int(window), float(scale), int(value_dim), float(softcap), extras.keep_first,
                                                   _ptr(extras.bias), extras.reach, _ptr(extras.sink), pooled.k_pages.data_ptr(),
                                                   pooled.v_pages.data_ptr(), pooled.block_table.data_ptr(),
                                                   pooled.block_table.shape[1], pooled.pool, _stream()))
        return out
    if extras:
        extras.check(heads)
        _check(lib, lib.nnis_attention_rows_more(q.data_ptr(), _code(q), out.data_ptr(), _code(out), k_pages.data_ptr(),
                                                 v_pages.data_ptr(), _code(k_pages), block_table.data_ptr(), block_table.shape[1],
                                                 tok_slot.data_ptr(), tok_pos.data_ptr(), tokens, heads, kv_heads, head_dim,
                                                 int(window), float(scale), int(value_dim), float(softcap), extras.keep_first,
                                                 _ptr(extras.bias), extras.reach, _ptr(extras.sink), _stream()))
        return out
    _check(lib, lib.nnis_attention_rows(q.data_ptr(), _code(q), out.data_ptr(), _code(out), k_pages.data_ptr(),
                                        v_pages.data_ptr(), _code(k_pages), block_table.data_ptr(), block_table.shape[1],
                                        tok_slot.data_ptr(), tok_pos.data_ptr(), tokens, heads, kv_heads, head_dim,
                                        int(window), float(scale), int(value_dim), float(softcap), _stream()))
    return out


# ---------------------------------------------------------------------------
# dispatch by operand types
# ---------------------------------------------------------------------------

class PackedWeight:
    """A bfloat16 weight [n, k] in the order the matrix-core products read it
    (``pack_weight``): strips of 16 rows, chunks of 64 k, both padded with
    zeros (and a strip to an odd number of chunks), a strip's chunk laid out
    as a wave's loads take it.  ``data`` is the
    flat packed storage; ``shape`` and ``dtype`` are the weight's own."""

    dtype = torch.bfloat16
    is_cuda = True

    def __init__(self, data: torch.Tensor, n: int, k: int):
        self.data = data
        self.shape = (int(n), int(k))

    @property
    def device(self):
        return self.data.device

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def is_contiguous(self) -> bool:
        return True


def packed_weight_elems(n: int, k: int) -> int:
    """Strips of 16 rows, each an odd number of chunks of 64 k (1024 elements) long."""
    return ((n + 15) // 16) * (((k + 63) // 64) | 1) * 1024


def packs(weight: torch.Tensor) -> bool:
    """Whether a weight is one that ``pack_weight`` takes."""
    return weight.is_cuda and weight.dim() == 2 and weight.dtype == torch.bfloat16 and weight.shape[1] % 8 == 0


def pack_weight(w: torch.Tensor) -> PackedWeight:
    """The packed copy of a bfloat16 weight [n, k] (K a multiple of 8) that
    ``gemm_bf16``, ``gemm_fused``, ``gemm_residual`` and ``gemm_scaled`` take."""
    _dev(w, "weight")
    if not packs(w):
        raise KernelError(f"pack_weight takes a bfloat16 matrix whose K is a multiple of 8, got {w.dtype} {tuple(w.shape)}")
    n, k = w.shape
    data = torch.empty(packed_weight_elems(n, k), dtype=torch.bfloat16, device=w.device)
    lib = core()
    _check(lib, lib.nnis_pack_weight(w.data_ptr(), data.data_ptr(), n, k, _stream()))
    return PackedWeight(data, n, k)


def _packed(w, what: str) -> None:
    if not isinstance(w, PackedWeight):
        raise KernelError(f"{what}: the weight must be packed (pack_weight) for the matrix-core kernels")


# Where the tiled product cuts K among blocks (few tiles, a long K) the parts meet in this scratch: 256 blocks
# of 64 x 64 sums at most.  Kept per device; calls on one device share it, so they follow one another on one
# stream.  It is made outside a graph capture only: a capture that finds none goes without the cut.
GEMM_WORKSPACE_BYTES = 4 << 20
_gemm_workspaces = {}
PAIR_COUNTS = 1024  # 32-bit words kept behind the workspace for the strips' counts


# Work that runs beside the main stream's (the branches of mixers side by side, on a second stream) has scratch
# of its own: a lane names whose.  Lane 0 is everybody's unless a part says otherwise around its launches.
_lane = 0


class lane:
    """``with ops.lane(1): ...``: the launches inside take lane 1's scratch (the products' workspace), so that they
    may run at the same time as launches outside that share the device."""

    def __init__(self, number: int):
        self.number, self.before = int(number), 0

    def __enter__(self):
        global _lane
        self.before, _lane = _lane, self.number
        return self

    def __exit__(self, *exc):
        global _lane
        _lane = self.before
        return False


def _gemm_workspace(device) -> Optional[torch.Tensor]:
    key = (device.type, device.index, _lane)
    held = _gemm_workspaces.get(key)
    if held is None and not torch.cuda.is_current_stream_capturing():
        # behind the workspace proper: the counts of the strips that two blocks share (`gemm_residual`), zero between calls
        held = _gemm_workspaces[key] = torch.zeros(GEMM_WORKSPACE_BYTES // 4 + PAIR_COUNTS, dtype=torch.float32, device=device)
    return held


def gemm_takes_pair(m: int, n: int, k: int) -> bool:
    """Whether ``gemm_residual`` gives a product of these sizes to two blocks a strip (the kernel whose blocks
    meet in the workspace and count in the words behind it)."""
    return bool(core().nnis_gemm_takes_pair(int(m), int(n), int(k), GEMM_WORKSPACE_BYTES))


def gemm_pair_counts(device) -> Optional[torch.Tensor]:
    """The strips' counts of the products with two blocks a strip on ``device`` (int32 [PAIR_COUNTS]; None
    before the first product there): every word is zero whenever no such product is running."""
    work = _gemm_workspace(torch.device(device))
    return None if work is None else work[GEMM_WORKSPACE_BYTES // 4:].view(torch.int32)


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, split: int = 0) -> torch.Tensor:
    """out[M, N] = x[M, K] @ w[N, K]^T on the matrix cores: bfloat16 operands,
    32-bit accumulation, bfloat16 or float32 output.  ``w``: a ``PackedWeight``."""
    _packed(w, "gemm_bf16")
    _dev(x, "x"), _dev(out, "out")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or out.shape != (m, n):
        raise KernelError(f"gemm: x {tuple(x.shape)} w {tuple(w.shape)} out {tuple(out.shape)} do not fit")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"gemm_bf16 takes bfloat16 operands, got {x.dtype} and {w.dtype}")
    lib = core()
    work = _gemm_workspace(x.device)
    _check(lib, lib.nnis_gemm_bf16(x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out), m, n, k, int(split), _ptr(work),
                                   GEMM_WORKSPACE_BYTES if work is not None else 0, _stream()))
    return out


EPILOGUE_STORE, EPILOGUE_SILU, EPILOGUE_ROPE = 0, 1, 2
# the gating epilogue with another activation than SiLU: the activation's code (``ACTIVATIONS``) rides above the epilogue's
EPILOGUE_GATE = {"silu": EPILOGUE_SILU, "gelu_tanh": EPILOGUE_SILU + 256 * 1, "relu": EPILOGUE_SILU + 256 * 2}
FUSED_MAX_TOKENS = 16  # beyond a tile of 16 tokens every wave re-reads too much of x: the separate kernels win


def gemm_fused(x_in: torch.Tensor, delta: Optional[torch.Tensor], x_out: Optional[torch.Tensor], norm_weight: torch.Tensor,
               eps: float, w: torch.Tensor, y: torch.Tensor, epilogue: int = EPILOGUE_STORE, rope: Optional[dict] = None,
               split: int = 0):
    """y = epilogue( W . rmsnorm(x_in + delta) ) for a few tokens (callers
    keep to ``FUSED_MAX_TOKENS``; the kernel itself takes up to 64), in one
    kernel; ``x_out`` receives x_in + delta.  ``epilogue``: store; SiLU(gate) *
    up for a weight of gate rows followed by up rows; or rotate-half RoPE with
    the write of keys and values into the cache (``rope``: cos, sin, tok_slot,
    tok_pos, k_pages, v_pages, block_table, heads, kv_heads, head_dim)."""
    _packed(w, "gemm_fused")
    m, k = x_in.shape
    n = w.shape[0]
    _dev(x_in, "x"), _dev(norm_weight, "norm weight"), _dev(y, "y")
    if x_in.dtype != torch.float32 or w.dtype != torch.bfloat16 or y.dtype != torch.bfloat16 or w.shape[1] != k:
        raise KernelError("gemm_fused: x must be float32 [m, k], the weight bfloat16 [n, k] and y bfloat16")
    if norm_weight.numel() != k:
        raise KernelError(f"gemm_fused: norm weight of {norm_weight.numel()} for width {k}")
    if delta is not None:
        _dev(delta, "delta"), _dev(x_out, "x_out")
        if delta.shape != x_in.shape or delta.dtype != torch.bfloat16 or x_out.shape != x_in.shape or x_out.dtype != torch.float32:
            raise KernelError("gemm_fused: delta must be bfloat16 and x_out float32, both shaped like x")
    r = _check_epilogue("gemm_fused", m, n, y, epilogue, rope)
    lib = core()
    bt = r.get("block_table")
    _check(lib, lib.nnis_gemm_fused(
        x_in.data_ptr(), _ptr(delta), _ptr(x_out) if delta is not None else None, norm_weight.data_ptr(), _code(norm_weight),
        float(eps), w.data_ptr(), m, n, k, int(epilogue), y.data_ptr(), _ptr(r.get("cos")), _ptr(r.get("sin")),
        r["cos"].shape[0] if r.get("cos") is not None else 0, _ptr(r.get("tok_slot")), _ptr(r.get("tok_pos")),
        _ptr(r.get("k_pages")), _ptr(r.get("v_pages")), _ptr(bt), bt.shape[1] if bt is not None else 0,
        r.get("heads", 0), r.get("kv_heads", 0), r.get("head_dim", 0), *_step_table_pointers(r), int(split), _stream()))
    return y


def _step_table_pointers(rope: dict):
    """(tok_cos, tok_sin, tok_page) of a rotating epilogue's ``tables`` (a ``StepTables``), or three nulls."""
    tables = rope.get("tables")
    if tables is None or tables.cos is None or tables.page is None:
        return None, None, None
    return tables.cos.data_ptr(), tables.sin.data_ptr(), tables.page.data_ptr()


def _check_epilogue(what: str, m: int, n: int, y: torch.Tensor, epilogue: int, rope: Optional[dict]) -> dict:
    """Checks y and the rotating epilogue's arguments against the sizes; returns the arguments (or {})."""
    expect = {EPILOGUE_STORE: (m, n), EPILOGUE_SILU: (m, n // 2)}.get(epilogue & 0xff if epilogue > 0 else epilogue)
    if epilogue >> 8 and ((epilogue & 0xff) != EPILOGUE_SILU or epilogue >> 8 not in ACTIVATIONS.values()):
        raise KernelError(f"{what}: unknown epilogue {epilogue}")
    r = rope or {}
    if epilogue == EPILOGUE_ROPE:
        expect = (m, r["heads"] * r["head_dim"])
        for name in ("cos", "sin", "tok_slot", "tok_pos"):
            _dev(r[name], name)
        if r["cos"].dtype != torch.float32 or r["cos"].shape != r["sin"].shape or r["cos"].shape[1] != r["head_dim"] // 2:
            raise KernelError(f"{what}: rotation tables must be float32 [positions, head_dim / 2]")
        if r["tok_slot"].dtype != torch.int32 or r["tok_pos"].dtype != torch.int32 or min(r["tok_slot"].numel(), r["tok_pos"].numel()) < m:
            raise KernelError(f"{what}: tok_slot / tok_pos must be int32 with one entry per token")
        tables = r.get("tables")
        if tables is not None and tables.cos is not None:
            if (tables.tokens < m or tables.cos.shape[1] != r["head_dim"] // 2 or tables.cos.dtype != torch.float32
                    or (r.get("k_pages") is not None and tables.page is None)):
                raise KernelError(f"{what}: the step's tables do not fit {m} tokens with heads of {r['head_dim']}")
        if r.get("k_pages") is not None:
            kp, vp, bt = r["k_pages"], r["v_pages"], r["block_table"]
            _dev(kp, "k_pages"), _dev(vp, "v_pages"), _dev(bt, "block_table")
            if (kp.dtype != torch.bfloat16 or vp.dtype != torch.bfloat16 or bt.dtype != torch.int32
                    or not _pages_fit(kp, vp, r["kv_heads"], r["head_dim"])):
                raise KernelError(f"{what}: cache pages must be bfloat16 in the cache's layout, the block table int32")
    if expect is None or tuple(y.shape) != expect or y.dtype != torch.bfloat16 or not y.is_contiguous():
        raise KernelError(f"{what}: y {tuple(y.shape)} {y.dtype} does not fit epilogue {epilogue} (expected bfloat16 {expect})")
    return r


# tiles of the tiled product (``tile`` of gemm_residual; 16 times as much as a ``split`` of gemm_bf16 / gemm_scaled)
TILE_64x128, TILE_64x64, TILE_256x256, TILE_256x192, TILE_128x128, TILE_256x128, TILE_128x192 = 2, 3, 4, 5, 6, 7, 8


def gemm_tile(m: int, n: int, k: int) -> int:
    """The tile (``TILE_*``) that the tiled kernel takes for a product of m rows with n weight rows of k."""
    return core().nnis_gemm_tile(int(m), int(n), int(k))


def gemm_residual_parts(m: int, n: int) -> int:
    """Rows of the ``ss`` scratch that ``gemm_residual`` may fill for these sizes."""
    return core().nnis_gemm_residual_parts(int(m), int(n))


def gemm_residual(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, gain: torch.Tensor, scaled: torch.Tensor,
                  ss: torch.Tensor, tile: int = 0) -> int:
    """The projection that ends a part of a pre-norm block: ``resid`` (float32
    [m, n]) takes x @ w^T in, in place, and the norm that follows is prepared:
    ``scaled`` = bfloat16(resid * gain) and, in ``ss`` [parts, m], parts of
    each row's sum of squares.  Returns how many parts were written; the
    norm's 1 / sqrt(mean + eps) is taken by ``gemm_scaled``, which reads them.
    ``x`` may be the ``KeyRuns`` of a decode attention (where ``fits``): the
    kernel then adds the runs up itself on its way.  ``tile`` (for tests and
    tuning): 0 lets the sizes choose, ``TILE_64x128``, ``TILE_64x64``,
    ``TILE_256x256``, ``TILE_256x192``, ``TILE_128x128``, ``TILE_256x128`` and
    ``TILE_128x192`` ask for the tiled kernel with that tile."""
    _packed(w, "gemm_residual")
    m, k = x.shape
    n = w.shape[0]
    runs = x if isinstance(x, KeyRuns) else None
    for t, what in ((x if runs is None else x.partial, "x"), (resid, "resid"), (gain, "gain"), (scaled, "scaled"),
                    (ss, "ss")):
        _dev(t, what)
        if not t.is_contiguous():
            raise KernelError(f"gemm_residual: {what} must be contiguous")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != k:
        raise KernelError("gemm_residual: x must be bfloat16 [m, k] and the weight bfloat16 [n, k]")
    if resid.dtype != torch.float32 or tuple(resid.shape) != (m, n) or scaled.dtype != torch.bfloat16 or tuple(scaled.shape) != (m, n):
        raise KernelError("gemm_residual: resid must be float32 [m, n] and scaled bfloat16 [m, n]")
    if gain.numel() != n:
        raise KernelError(f"gemm_residual: norm weight of {gain.numel()} for width {n}")
    if ss.dtype != torch.float32 or ss.numel() < m:
        raise KernelError("gemm_residual: ss must be float32 [rows, m] (gemm_residual_parts(m, n) rows are always enough)")
    lib = core()
    parts = ctypes.c_int(0)
    if runs is not None:
        if not runs.fits(n):
            raise KernelError("gemm_residual: these key runs are not taken; add them up first (KeyRuns.combine)")
        _check(lib, lib.nnis_gemm_residual_runs(runs.partial.data_ptr(), runs.runs, runs.heads, runs.head_dim, runs.tok_slot.data_ptr(),
                                                w.data_ptr(), resid.data_ptr(), gain.data_ptr(), _code(gain), scaled.data_ptr(),
                                                ss.data_ptr(), ss.numel() // m, m, n, ctypes.addressof(parts), _stream()))
        return parts.value
    work = _gemm_workspace(x.device)
    _check(lib, lib.nnis_gemm_residual(x.data_ptr(), w.data_ptr(), resid.data_ptr(), gain.data_ptr(), _code(gain),
                                       scaled.data_ptr(), ss.data_ptr(), ss.numel() // m, m, n, k, ctypes.addressof(parts),
                                       int(tile), _ptr(work), GEMM_WORKSPACE_BYTES if work is not None else 0,
                                       work.data_ptr() + GEMM_WORKSPACE_BYTES if work is not None else None, _stream()))
    return parts.value


def gemm_residual_tanh(x: torch.Tensor, w, resid: torch.Tensor, post, following, normed: torch.Tensor, ss: torch.Tensor) -> torch.Tensor:
    """The projection that ends a part of a block whose norms keep no
    statistics (y -> tanh(alpha y) weight + bias): ``resid`` (float32 [m, n])
    takes post(x @ w^T) in, in place, and ``normed`` (bfloat16 [m, n]) takes
    following(resid), the operand of the projection that comes next.
    ``post`` / ``following``: (alpha, weight, bias).  ``ss``: float32 scratch
    of ``gemm_residual_parts(m, n)`` rows of m (the kernels' sums of squares,
    which nobody reads here)."""
    _packed(w, "gemm_residual_tanh")
    m, k = x.shape
    n = w.shape[0]
    vectors = (post[1], post[2], following[1], following[2])
    for t, what in ((x, "x"), (resid, "resid"), (normed, "normed"), (ss, "ss")) + tuple((v, "norm vector") for v in vectors):
        _dev(t, what)
    if x.dtype != torch.bfloat16 or w.shape[1] != k:
        raise KernelError("gemm_residual_tanh: x must be bfloat16 [m, k] and the weight bfloat16 [n, k]")
    if resid.dtype != torch.float32 or tuple(resid.shape) != (m, n) or normed.dtype != torch.bfloat16 or tuple(normed.shape) != (m, n):
        raise KernelError("gemm_residual_tanh: resid must be float32 [m, n] and normed bfloat16 [m, n]")
    if any(v.numel() != n or v.dtype != vectors[0].dtype for v in vectors):
        raise KernelError(f"gemm_residual_tanh: the norms' vectors must have {n} entries of one type")
    if ss.dtype != torch.float32 or ss.numel() < gemm_residual_parts(m, n) * m:
        raise KernelError("gemm_residual_tanh: ss must be float32 with gemm_residual_parts(m, n) rows of m")
    lib = core()
    work = _gemm_workspace(x.device)
    _check(lib, lib.nnis_gemm_residual_tanh(x.data_ptr(), w.data_ptr(), resid.data_ptr(), post[1].data_ptr(), post[2].data_ptr(),
                                            float(post[0]), following[1].data_ptr(), following[2].data_ptr(), float(following[0]),
                                            _code(vectors[0]), normed.data_ptr(), ss.data_ptr(), ss.numel() // max(m, 1), m, n, k,
                                            _ptr(work), GEMM_WORKSPACE_BYTES if work is not None else 0,
                                            work.data_ptr() + GEMM_WORKSPACE_BYTES if work is not None else None, _stream()))
    return normed


def gemm_scaled(scaled: torch.Tensor, ss: torch.Tensor, parts: int, eps: float, w: torch.Tensor, y: torch.Tensor,
                epilogue: int = EPILOGUE_STORE, rope: Optional[dict] = None, split: int = 0) -> torch.Tensor:
    """y = epilogue( (W . scaled) / sqrt(sum of the parts of ss / k + eps) ):
    the second half of an RMSNorm whose first half ``gemm_residual`` took, with
    the epilogues of ``gemm_fused``."""
    _packed(w, "gemm_scaled")
    m, k = scaled.shape
    n = w.shape[0]
    for t, what in ((scaled, "scaled"), (ss, "ss"), (y, "y")):
        _dev(t, what)
    if scaled.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != k or not scaled.is_contiguous():
        raise KernelError("gemm_scaled: scaled must be bfloat16 [m, k] and the weight bfloat16 [n, k]")
    if ss.dtype != torch.float32 or parts <= 0 or ss.numel() < parts * m:
        raise KernelError("gemm_scaled: ss must be float32 [parts, m]")
    r = _check_epilogue("gemm_scaled", m, n, y, epilogue, rope)
    lib = core()
    work = _gemm_workspace(scaled.device)
    bt = r.get("block_table")
    _check(lib, lib.nnis_gemm_scaled(
        scaled.data_ptr(), ss.data_ptr(), int(parts), float(eps), w.data_ptr(), m, n, k, int(epilogue), y.data_ptr(),
        _ptr(r.get("cos")), _ptr(r.get("sin")), r["cos"].shape[0] if r.get("cos") is not None else 0, _ptr(r.get("tok_slot")),
        _ptr(r.get("tok_pos")), _ptr(r.get("k_pages")), _ptr(r.get("v_pages")), _ptr(bt), bt.shape[1] if bt is not None else 0,
        r.get("heads", 0), r.get("kv_heads", 0), r.get("head_dim", 0), *_step_table_pointers(r), int(split), _ptr(work),
        GEMM_WORKSPACE_BYTES if work is not None else 0, _stream()))
    return y


_unit_rows = {}  # per device: zeros that stand for rows whose scale is one
UNIT_ROWS_MOST = 1 << 16


def gated_linear(x: torch.Tensor, weight, out: torch.Tensor, activation: str) -> torch.Tensor:
    """out = act(x @ gate^T) * (x @ up^T) for a packed weight whose first half
    of rows is the gate: the product with the gating in its epilogue, on plain
    rows (``gemm_scaled`` with a row scale of one: sums of squares of zero and
    an eps of one).  Up to ``UNIT_ROWS_MOST`` rows; call ``unit_rows(device)``
    once outside any graph capture before the first use."""
    m = x.shape[0]
    if m > UNIT_ROWS_MOST:
        raise KernelError(f"gated_linear: up to {UNIT_ROWS_MOST} rows are taken, got {m}")
    return gemm_scaled(x, unit_rows(x.device)[:m].view(1, m), 1, 1.0, weight, out, EPILOGUE_GATE[activation])


def unit_rows(device) -> torch.Tensor:
    device = torch.device(device)
    key = (device.type, device.index)
    held = _unit_rows.get(key)
    if held is None:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("gated_linear: its rows of zeros would have to be made inside a graph capture")
        held = _unit_rows[key] = torch.zeros(UNIT_ROWS_MOST, dtype=torch.float32, device=device)
    return held


def linear(x: torch.Tensor, weight, out: torch.Tensor) -> torch.Tensor:
    """out = x @ weight^T.  A packed weight (bfloat16) takes the matrix-core
    kernels; a weight as the checkpoint has it (32-bit, or a width the 16-byte
    loads cannot take) the ordered 32-bit product."""
    if isinstance(weight, PackedWeight):
        if x.dtype != torch.bfloat16 or x.data_ptr() % 16 != 0 or out.data_ptr() % 16 != 0:
            raise KernelError(f"linear: a packed weight multiplies bfloat16 rows on 16-byte boundaries, got {x.dtype}")
        return gemm_bf16(x, weight, out)
    return gemm_ordered(x, weight, out)


def _check_pages(q, out, k_pages, v_pages, block_table, heads, kv_heads, head_dim, value_dim=None):
    tokens = q.shape[0]
    value_dim = value_dim or head_dim
    if q.shape != (tokens, heads * head_dim) or out.shape != (tokens, heads * value_dim):
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {heads} heads of {head_dim} "
                          f"with values of {value_dim}")
    if not _pages_fit(k_pages, v_pages, kv_heads, head_dim, value_dim):
        raise KernelError(f"attention: page shapes {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not fit")
    if block_table.dtype != torch.int32 or block_table.dim() != 2:
        raise KernelError("attention: block_table must be int32 [slots, pages]")
    for t, what in ((q, "q"), (out, "out"), (k_pages, "k_pages"), (v_pages, "v_pages")):
        _dev(t, what)
        if t.dtype != torch.bfloat16:
            raise KernelError(f"attention: the matrix-core kernels take bfloat16, {what} is {t.dtype}")


def prefill_tile_rows(heads: int, kv_heads: int, head_dim: int, columns: int = 0, value_dim=None, softcap=0.0, extras=None, pooled=None) -> int:
    """Query rows per work item of ``attention_prefill_bf16`` for these sizes.
    ``columns``: the most 16-column tiles (query tiles x heads of a group) a
    wave carries; 0 for as many as the head size allows."""
    return attention_module(head_dim, value_dim, softcap, extras, pooled).nnis_attention_prefill_tile_rows(heads, kv_heads, columns)


def prefill_max_waves(heads: int, kv_heads: int, head_dim: int, columns: int = 0, value_dim=None, softcap=0.0, extras=None, pooled=None) -> int:
    return attention_module(head_dim, value_dim, softcap, extras, pooled).nnis_attention_prefill_max_waves(heads, kv_heads, columns)


def attention_prefill_bf16(q, out, k_pages, v_pages, block_table, tile_seq, tile_row0, seq_slot, seq_start, seq_pos0,
                           heads, kv_heads, head_dim, scale, window=0, waves=1, columns=0, value_dim=None, softcap=0.0,
                           extras: Optional[ScoreExtras] = None, pooled: Optional[PooledBlocks] = None):
    """Causal attention of whole runs of new tokens over the cache, on the
    matrix cores.  ``tile_seq``/``tile_row0`` (int32) name, per work item, a
    sequence of the step and the first of ``prefill_tile_rows`` rows of its
    new tokens; ``seq_start`` [batch + 1] gives each sequence's packed rows."""
    _check_pages(q, out, k_pages, v_pages, block_table, heads, kv_heads, head_dim, value_dim)
    for t in (tile_seq, tile_row0, seq_slot, seq_start, seq_pos0):
        _dev(t, "step metadata")
        if t.dtype != torch.int32:
            raise KernelError("attention: step metadata must be int32")
    tiles = tile_seq.numel()
    if tile_row0.numel() != tiles or seq_start.numel() != seq_slot.numel() + 1 or seq_pos0.numel() != seq_slot.numel():
        raise KernelError("attention: step metadata arrays do not fit each other")
    lib = attention_module(head_dim, value_dim, softcap, extras, pooled)
    if pooled is not None:
        extras = extras or ScoreExtras()
        extras.check(heads)
        pooled.check(k_pages, v_pages, kv_heads, head_dim, value_dim or head_dim, window)
        _check(lib, lib.nnis_attention_prefill_bf16_pooled(
            q.data_ptr(), out.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1],
            tile_seq.data_ptr(), tile_row0.data_ptr(), tiles, seq_slot.data_ptr(), seq_start.data_ptr(), seq_pos0.data_ptr(), heads,
            kv_heads, head_dim, int(window), float(scale), int(waves), int(columns), float(softcap), extras.keep_first,
            _ptr(extras.bias), extras.reach, _ptr(extras.sink), pooled.k_pages.data_ptr(), pooled.v_pages.data_ptr(),
            pooled.block_table.data_ptr(), pooled.block_table.shape[1], pooled.pool, _stream()))
        return out
    if extras:
        extras.check(heads)
        _check(lib, lib.nnis_attention_prefill_bf16_more(
            q.data_ptr(), out.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1],
            tile_seq.data_ptr(), tile_row0.data_ptr(), tiles, seq_slot.data_ptr(), seq_start.data_ptr(), seq_pos0.data_ptr(), heads,
            kv_heads, head_dim, int(window), float(scale), int(waves), int(columns), float(softcap), extras.keep_first,
            _ptr(extras.bias), extras.reach, _ptr(extras.sink), _stream()))
        return out
    _check(lib, lib.nnis_attention_prefill_bf16(q.data_ptr(), out.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
                                                block_table.data_ptr(), block_table.shape[1], tile_seq.data_ptr(),
                                                tile_row0.data_ptr(), tiles, seq_slot.data_ptr(), seq_start.data_ptr(),
                                                seq_pos0.data_ptr(), heads, kv_heads, head_dim, int(window), float(scale),
                                                int(waves), int(columns), float(softcap), _stream()))
    return out


def attention_decode_bf16(q, out, k_pages, v_pages, block_table, tok_slot, tok_pos, heads, kv_heads, head_dim, scale,
                          window=0, splits=1, partial=None, waves=1, kernel="auto", keep_runs=False, token_pages=None,
                          value_dim=None, softcap=0.0, extras: Optional[ScoreExtras] = None, pooled: Optional[PooledBlocks] = None):
    """One query token per sequence over its cached keys.  The keys are cut
    into ``splits`` runs, each a block of ``waves`` waves that deal its pages
    among themselves and merge in LDS; the runs are summed by a second kernel.
    ``partial``: float32 scratch of tokens * heads * splits * (head_dim + 4)
    when splits > 1 (``decode_scratch`` keeps one per device).  ``keep_runs``
    (with splits > 1): the second kernel is left out and a ``KeyRuns`` is
    returned in place of ``out`` -- the projection that follows adds the runs
    up itself (``gemm_residual``), or ``KeyRuns.combine()`` does.  ``kernel``:
    "keys" (keys on lanes; groups of up to 4 heads of up to 128 channels),
    "columns" (heads in the columns of a tile; any group the head size
    carries) or "auto", which takes "keys" where it fits.  ``token_pages``
    (int32 [tokens, pages], ``StepTables.pages``): each token's sequence's
    pages, read in place of the block table's row of the token's slot."""
    _check_pages(q, out, k_pages, v_pages, block_table, heads, kv_heads, head_dim, value_dim)
    value_dim = value_dim or head_dim
    tokens = q.shape[0]
    table = block_table
    if token_pages is not None:
        _dev(token_pages, "token_pages")
        if token_pages.dtype != torch.int32 or token_pages.dim() != 2 or token_pages.shape[0] < tokens:
            raise KernelError("attention: token_pages must be int32 [tokens, pages]")
        table = token_pages
    for t in (tok_slot, tok_pos):
        _dev(t, "step metadata")
        if t.dtype != torch.int32 or t.numel() < tokens:
            raise KernelError("attention: tok_slot / tok_pos must be int32 with one entry per token")
    if splits > 1:
        if partial is None or partial.dtype != torch.float32 or partial.numel() < tokens * heads * splits * (value_dim + 4):
            raise KernelError("attention: splits need float32 scratch of tokens * heads * splits * (value channels + 4)")
        _dev(partial, "partial")
    lib = attention_module(head_dim, value_dim, softcap, extras, pooled)
    if pooled is not None:
        extras = extras or ScoreExtras()
        extras.check(heads)
        pooled.check(k_pages, v_pages, kv_heads, head_dim, value_dim, window)
        _check(lib, lib.nnis_attention_decode_bf16_pooled(
            q.data_ptr(), out.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), table.data_ptr(), table.shape[1],
            tok_slot.data_ptr(), tok_pos.data_ptr(), tokens, heads, kv_heads, head_dim, int(window), float(scale), int(splits),
            int(waves), _ptr(partial) if splits > 1 else None, _DECODE_KERNELS["columns"], 0 if (keep_runs and splits > 1) else 1,
            1 if token_pages is not None else 0, float(softcap), extras.keep_first, _ptr(extras.bias), extras.reach,
            _ptr(extras.sink), pooled.k_pages.data_ptr(), pooled.v_pages.data_ptr(), pooled.block_table.data_ptr(),
            pooled.block_table.shape[1], pooled.pool, _stream()))
    elif extras:
        extras.check(heads)
        _check(lib, lib.nnis_attention_decode_bf16_more(
            q.data_ptr(), out.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), table.data_ptr(), table.shape[1],
            tok_slot.data_ptr(), tok_pos.data_ptr(), tokens, heads, kv_heads, head_dim, int(window), float(scale), int(splits),
            int(waves), _ptr(partial) if splits > 1 else None, _DECODE_KERNELS[kernel], 0 if (keep_runs and splits > 1) else 1,
            1 if token_pages is not None else 0, float(softcap), extras.keep_first, _ptr(extras.bias), extras.reach,
            _ptr(extras.sink), _stream()))
    else:
        _check(lib, lib.nnis_attention_decode_bf16(q.data_ptr(), out.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(),
                                                   table.data_ptr(), table.shape[1], tok_slot.data_ptr(),
                                                   tok_pos.data_ptr(), tokens, heads, kv_heads, head_dim, int(window),
                                                   float(scale), int(splits), int(waves), _ptr(partial) if splits > 1 else None,
                                                   _DECODE_KERNELS[kernel], 0 if (keep_runs and splits > 1) else 1,
                                                   1 if token_pages is not None else 0, float(softcap), _stream()))
    if keep_runs and splits > 1:
        return KeyRuns(partial, int(splits), tokens, heads, value_dim, tok_slot, out, lib)
    return out


# Up to this many tokens a decode step leaves its runs of keys to the output projection; beyond, every block of
# the projection making the same activations again costs more than the kernel between the two.
KEY_RUNS_MOST_TOKENS = 4


class KeyRuns:
    """What the decode attention leaves when it cuts the keys into runs and is
    told not to add them up: per (token, head, run) the run's outputs, its
    softmax reference and its sum, in ``partial`` (the device's decode scratch:
    valid until the next decode attention on this device).  A stand-in for the
    attention's output [tokens, heads * head_dim] in bfloat16."""

    dtype = torch.bfloat16

    def __init__(self, partial, runs, tokens, heads, head_dim, tok_slot, out, module=None):
        """``head_dim``: the channels of a head's output (its values'); ``module``: the attention module that left the runs."""
        self.partial, self.runs, self.tokens, self.heads, self.head_dim = partial, runs, tokens, heads, head_dim
        self.tok_slot, self.out, self.module = tok_slot, out, module
        self.shape = (tokens, heads * head_dim)

    def fits(self, rows_out: int) -> bool:
        """Whether ``gemm_residual`` takes these runs for a weight of ``rows_out`` rows."""
        return bool(core().nnis_gemm_residual_runs_fits(self.tokens, int(rows_out), self.heads, self.head_dim, self.runs))

    def combine(self) -> torch.Tensor:
        """The attention's output, added up by the kernel of its own."""
        lib = self.module or attention_module(self.head_dim)
        _check(lib, lib.nnis_attention_combine(self.partial.data_ptr(), self.out.data_ptr(), self.tok_slot.data_ptr(), self.tokens,
                                               self.heads, self.head_dim, self.runs, _stream()))
        return self.out


_DECODE_KERNELS = {"auto": 0, "columns": 1, "keys": 2}
_decode_scratch = {}  # per device: the scratch in use


def decode_scratch(device, floats: int) -> torch.Tensor:
    """Scratch of the split decode attention, kept per device.  Calls on one
    device share it, so they must follow one another on one stream.  A call
    that needs more gets a larger tensor, made outside a graph capture only
    (the run that warms a graph up sizes it), and the smaller one is let go:
    kernels already on the stream are ahead of whoever gets its memory next,
    and a captured graph, which has the address it was captured with baked in
    and goes on writing there on every replay, holds the tensor itself for as
    long as it lives (``Part.held_buffers``, ``engine/graph.py``)."""
    key = (device.type, device.index)
    held = _decode_scratch.get(key)
    if held is None or held.numel() < floats:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("attention: the decode scratch would have to grow inside a graph capture")
        held = _decode_scratch[key] = torch.empty(max(floats, 2 * held.numel() if held is not None else 1 << 16),
                                                   dtype=torch.float32, device=device)
    return held


def decode_scratch_held(device):
    """The scratch a decode attention launched now would use (None: none made yet)."""
    return _decode_scratch.get((device.type, device.index))


def decode_max_waves(heads: int, kv_heads: int, head_dim: int, value_dim=None, softcap=0.0, extras=None, pooled=None) -> int:
    return attention_module(head_dim, value_dim, softcap, extras, pooled).nnis_attention_decode_max_waves(heads, kv_heads)


def decode_plan(batch: int, kv_heads: int, longest: int, max_waves: int = 4, width: int = 0):
    """(splits, waves) of a decode step's attention.  A block of 4 waves deals
    a sequence's pages among its waves.  Cutting the keys into runs for more
    blocks costs a second kernel that sums the runs (dearer the more runs), so
    it pays only from about 9 pages on; then a wave gets 1 to 2 pages, in at
    most 8 runs and about a thousand waves on the chip.  Powers of two.
    ``width`` (query heads x head size, 0: unknown) says what a run costs to
    sum: beyond 1024 runs pay from 17 pages on and a wave gets 2 to 4 pages
    (32 heads of 64, 128 to 2k keys, tokens/s with the one rule and the other:
    batch 8 on 4 key-value heads 5,654 against 5,497, batch 1 862 against 852;
    batch 1 on 32 key-value heads 700 against 682).
    Measured on 9 query / 3 key-value heads of 64 (microseconds a layer, runs
    of 1/2/4/8/16): batch 1 at 1k keys 7.9/8.3/8.7/10.7, at 8k 30/20/15/14/17;
    batch 8 at 2k 11.6/11.0/9.5/9.3/13.6; batch 32 at 4k 27/25/31/34/45.  And
    on whole decode steps of 30 such layers (milliseconds, runs of 1/2/4/8 with
    4 waves): batch 1 at 1k keys 0.839/0.822/0.790/0.775, at 128 to 2k
    0.957/0.882/0.823/0.790, at 256 keys 0.724/0.742/0.741/0.749; batch 8 at 1k
    0.943/0.952/0.919/0.914, at 128 to 2k 1.051/0.968/0.910/0.890, at 512 keys
    0.874/0.900/0.881/0.893."""
    pages = (longest + 63) // 64
    waves = 1
    while waves * 2 <= min(max_waves, pages):
        waves *= 2
    splits = 1
    first, each = (8, 4) if 0 < width <= 1024 else (16, 8)  # runs from more than `first` pages on, about `each` pages a run
    if pages > first:
        wanted = min(8, (pages + each - 1) // each)
        room = max(1, 1024 // max(1, batch * kv_heads * waves))
        while splits * 2 <= room and splits < wanted:
            splits *= 2
    if splits == 1 and batch * kv_heads >= 2048:
        # eight and more blocks a compute unit: two waves a block read as fast as four or faster (batch 64 on 32
        # key-value heads of 64, whole steps: 1,000 to 1,100 keys each 16,230 tokens/s against 15,900, 128 to 2k
        # 15,620 either way); at four blocks a unit four waves are faster (batch 32: 12,010 against 11,600)
        waves = min(waves, 2)
    return splits, waves


# The prefill attention's plan: the waves of a block, and the most column tiles (query tiles x heads of a group) a
# wave carries, 0 for as many as the head size allows.  Fewer columns make more and lighter work items, which a step
# of few tokens needs to fill the chip, and read keys and values more often, which a long one pays for.  Measured on
# one sequence, microseconds a layer, as it was (2, 4, 8 waves from 128, 512, 1,024 tokens on, always the widest
# tiles) against these plans: 9/3 heads of 64 at 128 / 512 / 768 tokens 16.9 / 11.7 / 11.0 against 9.8 / 9.7 / 10.1;
# 32/32 heads at 128 / 512 / 1,024 10.9 / 12.9 / 22.5 against 9.4 / 11.1 / 16.7; 32/4 heads 10.3 / 12.1 / 22.3
# against 9.6 / 10.8 / 17.3.  From 1,024 tokens on 9/3 heads are fastest with the widest tiles and 8 waves (12.9
# against 13.3), from 1,536 on all three are (9/3: 14.9 against 22.9 with two columns).  Whole prompt steps, ms:
# TinyLlama shape 128 / 1,024 tokens 1.68 / 4.31 -> 1.60 / 4.19, 135M shape 128 / 256 1.04 / 1.32 -> 0.99 / 1.23.
PREFILL_MANY_ROWS = 65536  # rows x query heads from which a step has work items enough for the widest tiles
PREFILL_SOME_ROWS = 16384  # ... from which a step of 1,024 to 1,279 tokens still gains by two columns
# Items of four columns (up to 64 channels, any group but 3) merge the states of 8 waves through 72 KB of LDS: worth it
# while a step's items are few (16 heads of 64 at 2,048 tokens 26 us a layer against 37 with 4 waves, 16/4 heads of 48
# 25 against 39; 32 heads at 1,024 tokens 21 against 25), not beyond (32 heads at 1,536 tokens 41 against 35, 64/8 heads
# at 2,048 83 against 73).
PREFILL_EIGHT_WAVES_MOST = 40960


def prefill_plan(longest: int, rows: int, heads: int, head_dim: int = 64, kv_heads: int = 0):
    """(waves of a block, column option) of the prefill attention for a step of ``rows`` rows (what the engine
    plans for: a step's tokens rounded up as a replayed step's are) whose longest sequence has ``longest``
    (``kv_heads``: 0 for as many as ``heads``)."""
    plan_class = prefill_plan_class(longest)
    size = rows * heads
    # A step with work items for about twice the waves that the chip holds (two a SIMD up to 64 channels, one
    # beyond; an item is 16 rows x 4, 2 or 1 columns) gives each item to one wave, which needs no merge and pays an
    # item's first loads once.  One sequence, microseconds a layer with one wave against the plan by length: 32
    # heads of 64 at 8,192 tokens 349 against 467; 64/8 heads of 64 at 4,096 180 against 243; 32/8 heads of 128 at
    # 2,048 66 against 102, at 8,192 833 against 1,306; 16 heads of 96 at 8,192 259 against 349.  Up to 64 channels a
    # step of half that size has the items with two columns: 32 heads at 4,096 tokens 119 against 137, 64/8 heads at
    # 2,048 64 against 74, 16 heads at 8,192 213 against 243, and from three eighths on 32 heads at 3,072 83 against
    # 93 -- where two columns divide a group's heads (of 9/3 heads they would leave a quarter of the columns empty:
    # 227 against 145 at 8,192; 24/8 heads of 64 at 8,192 tokens have items of three columns for twice the chip's
    # waves: 276 with one wave an item against 345).  At a quarter (32 heads at 2,048 tokens) the kernel alone took 49
    # against 47 to 56 and whole prompts 2 to 3% longer: not taken there.
    # With fewer items the waves of a block deal an item's keys: 9/3 heads of 64 at 8,192 tokens 141 with 8 waves,
    # 193 with one.
    group = heads // kv_heads if kv_heads else 1
    wide = (3 if group == 3 else 4) if head_dim <= 64 else (2 if head_dim <= 128 else 1)  # (a group of 3 heads fills 3 columns)
    # (Since the waves of a block that holds a long item and a short one are shared out by their pages also in
    # odd numbers -- 3 + 1 of 4 -- the blocks of 4 waves hold out longer: 32 heads of 64 at 3,072 tokens 68 us
    # against 78 with one wave an item of two columns, equal at 4,096; 32/8 heads of 128 at 2,048 tokens 58
    # against 66 with one wave an item, at 4,096 200 against 179.)
    many = 2 * (2048 if head_dim <= 64 else 1024) * 16 * wide
    if size >= (2 * many if 64 < head_dim <= 128 else many):
        return 1, 0
    if head_dim <= 64 and 2 * size >= many and (group == 1 or group % 2 == 0):
        return 1, 2
    waves = (1, 2, 4, 8, 8)[plan_class]
    if waves == 8 and head_dim <= 64 and group != 3 and size > PREFILL_EIGHT_WAVES_MOST:
        waves = 4
    if plan_class == 0 or plan_class == 4 or size >= PREFILL_MANY_ROWS:
        return waves, 0
    if plan_class == 3:
        if size < PREFILL_SOME_ROWS:
            return 8, 0
        return (4, 0) if group == 3 else (4, 2)  # (two columns would leave a group of 3 heads a quarter of them empty)
    return waves, plan_class  # 2 waves and one column from 128 tokens on, 4 waves and two columns from 512 on


def prefill_plan_class(longest: int) -> int:
    """Steps whose longest sequence falls into the same class launch the same prefill attention kernels
    (``attention`` picks the waves of a block, and the column option, by these thresholds)."""
    return 4 if longest >= 1280 else (3 if longest >= 1024 else (2 if longest >= 512 else (1 if longest >= 128 else 0)))


PREFILL_CLASS_LENGTH = (1, 128, 512, 1024, 1280)  # a length of each class


def _prefill_tile_arrays(new_tokens, first_positions, rows: int):
    """``prefill_tile_items`` as two int64 arrays (a step of thousands of tokens has hundreds of tiles: arrays,
    not a loop, while the GPU waits for the host)."""
    import numpy as np

    counts, pos0 = np.asarray(new_tokens, dtype=np.int64), np.asarray(first_positions, dtype=np.int64)
    tiles = (counts + rows - 1) // rows  # of each sequence
    seq = np.repeat(np.arange(counts.size, dtype=np.int64), tiles)
    row0 = (np.arange(int(tiles.sum()), dtype=np.int64) - np.repeat(np.cumsum(tiles) - tiles, tiles)) * rows
    last_key = pos0[seq] + np.minimum(row0 + rows, counts[seq])  # one beyond the last key that the tile's last row reads
    order = np.lexsort((-row0, -seq, -last_key))  # most keys first; among equals the later sequence, the later row
    return seq[order], row0[order]


def prefill_tile_items(new_tokens, first_positions, rows: int):
    """Work items (sequence of the step, first row) of a prefill step for tiles of ``rows`` query rows: those
    with the most keys first."""
    seq, row0 = _prefill_tile_arrays(new_tokens, first_positions, rows)
    return seq.tolist(), row0.tolist()


NO_ROWS = 1 << 24  # first row of a work item that has none: it lies beyond any sequence's tokens


def prefill_tile_list(new_tokens, first_positions, padded, rows: int):
    """``prefill_tile_items`` as one int32 array [2, items] (row 0 the sequences, row 1 the first rows), the form in
    which a step keeps its work lists (``StepContext.lists``).  ``padded``: None, or (sequences, rows of the step)
    of a step that runs from fixed buffers: the list then has as many items as any step of that shape can have
    (rows of the step / rows of a tile + sequences), those beyond the step's own with no rows."""
    import numpy as np

    seqs, row0s = _prefill_tile_arrays(new_tokens, first_positions, rows)
    count = len(seqs)
    if padded is not None:
        count = padded[1] // rows + padded[0]
        if len(seqs) > count:
            raise KernelError(f"{len(seqs)} work items for a step of {padded[0]} sequences and {padded[1]} rows")
    out = np.empty((2, count), dtype=np.int32)
    out[0, :len(seqs)], out[0, len(seqs):] = seqs, 0
    out[1, :len(seqs)], out[1, len(seqs):] = row0s, NO_ROWS
    return out


def attention(q: torch.Tensor, out: torch.Tensor, view, ctx, heads: int, kv_heads: int, head_dim: int, scale: float,
              window: int = 0, keep_runs: bool = False, tables: Optional[StepTables] = None, plan=None,
              value_dim: Optional[int] = None, softcap: float = 0.0, extras: Optional[ScoreExtras] = None,
              pooled: Optional[PooledBlocks] = None):
    """Attention of the step's tokens over the cache ``view``: bfloat16 with a
    head size in steps of 16 runs on the matrix cores (one kernel for single
    tokens, one for runs of tokens); anything else takes the 32-bit kernel.
    ``keep_runs``: a decode step whose keys are cut into runs may return them
    as ``KeyRuns`` instead of the output (see ``attention_decode_bf16``).
    ``plan``: (runs, waves) of a step of single tokens (``decode_plan``), or
    (waves, columns) of a step of prompts (``prefill_plan``); None: as those
    functions choose for the step's planned sizes."""
    value_dim = value_dim or head_dim
    fast = attention_on_matrix_cores(q.dtype, view.k_pages.dtype, head_dim, value_dim, softcap, extras)
    size = max(head_dim, value_dim)  # what a wave's registers are sized by
    if fast and ctx.decode and heads // kv_heads <= 16 * (4 if size <= 64 else (2 if size <= 128 else 1)):
        splits, waves = plan or decode_plan(ctx.batch, kv_heads, ctx.planned_len, width=heads * value_dim)
        waves = min(waves, decode_max_waves(heads, kv_heads, head_dim, value_dim, softcap, extras, pooled))
        partial = None
        if splits > 1:
            partial = decode_scratch(q.device, q.shape[0] * heads * splits * (value_dim + 4))
        return attention_decode_bf16(q, out, view.k_pages, view.v_pages, view.block_table, ctx.tok_slot, ctx.tok_pos, heads,
                                     kv_heads, head_dim, scale, window, splits, partial, waves,
                                     keep_runs=keep_runs and q.shape[0] <= KEY_RUNS_MOST_TOKENS,
                                     token_pages=tables.pages if tables is not None else None, value_dim=value_dim, softcap=softcap,
                                     extras=extras, pooled=pooled)
    if fast and not ctx.decode:
        # A tile's keys are a chain of dependent loads: the longest tile sets the kernel's time.  The waves of
        # a block deal the keys among themselves (their merge lives in LDS).
        waves, columns = plan or prefill_plan(ctx.planned_len, ctx.planned_rows, heads, size, kv_heads)
        waves = min(waves, prefill_max_waves(heads, kv_heads, head_dim, columns, value_dim, softcap, extras, pooled))
        rows = prefill_tile_rows(heads, kv_heads, head_dim, columns, value_dim, softcap, extras, pooled)
        tiles = ctx.lists.device_list(("attention_tiles", rows), lambda new, first, padded: prefill_tile_list(new, first, padded, rows))
        return attention_prefill_bf16(q, out, view.k_pages, view.v_pages, view.block_table, tiles[0], tiles[1],
                                      ctx.seq_slot, ctx.seq_start, ctx.seq_pos0, heads, kv_heads, head_dim, scale, window,
                                      waves, columns, value_dim, softcap, extras, pooled)
    return attention_rows(q, out, view.k_pages, view.v_pages, view.block_table, ctx.tok_slot, ctx.tok_pos, heads,
                          kv_heads, head_dim, scale, window, value_dim, softcap, extras, pooled)


def attention_on_matrix_cores(q_dtype, cache_dtype, head_dim: int, value_dim: Optional[int] = None, softcap: float = 0.0,
                              extras: Optional[ScoreExtras] = None) -> bool:
    """Whether ``attention`` takes the matrix-core kernels for these types and sizes (else the 32-bit row kernel)."""
    return (q_dtype == torch.bfloat16 and cache_dtype == torch.bfloat16 and head_dim % 16 == 0
            and (value_dim or head_dim) % 16 == 0 and max(head_dim, value_dim or head_dim) <= ATTENTION_MOST_CHANNELS)


def sample(logits: torch.Tensor, weights: torch.Tensor, row_slot: torch.Tensor, rng: torch.Tensor,
           temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor, out: torch.Tensor, by_slot: bool = False,
           best: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Seeded sampling per row; rows whose slot is negative are skipped (their
    ``out`` stays as it is).  ``rng`` is int64 [slots] holding each sequence's
    SplitMix64 state; ``weights`` is float64 scratch of at least [rows, vocab].
    ``temperature``, ``top_k`` and ``top_p`` hold a value per row, or, with
    ``by_slot``, per slot (like ``rng``).  ``best`` (int32 [rows], may be
    ``out``) holds an index of each row's maximum where the caller has it
    (``argmax``); without it the maxima are found here.  A row with a
    non-finite logit gets -1."""
    for t, what in ((logits, "logits"), (weights, "weights"), (row_slot, "row_slot"), (rng, "rng"),
                    (temperature, "temperature"), (top_k, "top_k"), (top_p, "top_p"), (out, "out")):
        _dev(t, what)
    rows, vocab = logits.shape
    if logits.dtype != torch.float32 or weights.dtype != torch.float64 or weights.numel() < rows * vocab:
        raise KernelError("sample: logits must be float32 and weights float64 scratch of [rows, vocab]")
    if rng.dtype != torch.int64 or row_slot.dtype != torch.int32 or top_k.dtype != torch.int32 or out.dtype != torch.int32:
        raise KernelError("sample: rng must be int64; row_slot, top_k and out int32")
    if temperature.dtype != torch.float32 or top_p.dtype != torch.float32:
        raise KernelError("sample: temperature and top_p must be float32")
    if min(row_slot.numel(), out.numel()) < rows:
        raise KernelError("sample: per-row arrays are shorter than the rows")
    needed = rng.numel() if by_slot else rows
    if min(temperature.numel(), top_k.numel(), top_p.numel()) < needed:
        raise KernelError("sample: temperature, top_k and top_p need a value per " + ("slot" if by_slot else "row"))
    if best is None:
        best = argmax(logits, torch.empty(rows, dtype=torch.int32, device=logits.device))
    else:
        _dev(best, "best")
        if best.dtype != torch.int32 or best.numel() < rows:
            raise KernelError("sample: best must be int32 [rows]")
    lib = core()
    _check(lib, lib.nnis_sample(logits.data_ptr(), weights.data_ptr(), rows, vocab, row_slot.data_ptr(), rng.data_ptr(),
                                temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), 1 if by_slot else 0,
                                best.data_ptr(), out.data_ptr(), _stream()))
    return out


# ---------------------------------------------------------------------------
# a residual kept as several streams; branches side by side; activations
# ---------------------------------------------------------------------------

def embed_pair(ids: torch.Tensor, tok_slot: torch.Tensor, tok_pos: torch.Tensor, table: torch.Tensor, pairs: torch.Tensor,
               mul_prev: int, mul_cur: int, last_token: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[c, t, :] = table[ids[t]] + pairs[row] for every copy c of ``out`` [copies, tokens, width] (32-bit), with
    row = (token before * mul_prev + ids[t] * mul_cur) % (rows of ``pairs`` - 1), or the last row of ``pairs`` for a
    sequence's first token.  ``last_token`` (int32 [slots]) holds, per slot, the last token of the step before, and
    is left holding this step's.  Padding rows (negative slot, id outside the table) are zero."""
    for t, what in ((ids, "ids"), (tok_slot, "tok_slot"), (tok_pos, "tok_pos"), (table, "table"), (pairs, "pairs"),
                    (last_token, "last_token"), (out, "out")):
        _dev(t, what)
    copies, tokens, width = out.shape
    if out.dtype != torch.float32 or table.dim() != 2 or pairs.dim() != 2 or table.shape[1] != width or pairs.shape[1] != width:
        raise KernelError(f"embed_pair: tables {tuple(table.shape)} / {tuple(pairs.shape)} do not fit out {tuple(out.shape)} {out.dtype}")
    if pairs.shape[0] < 2:
        raise KernelError("embed_pair: the table of pairs needs at least one bucket and the row of a first token")
    for t in (ids, tok_slot, tok_pos):
        if t.dtype != torch.int32 or t.numel() < tokens:
            raise KernelError("embed_pair: ids, tok_slot and tok_pos must be int32 with one entry per token")
    if last_token.dtype != torch.int32:
        raise KernelError("embed_pair: last_token must be int32 [slots]")
    lib = core()
    _check(lib, lib.nnis_embed_pair(ids.data_ptr(), tok_slot.data_ptr(), tok_pos.data_ptr(), tokens, table.data_ptr(), _code(table),
                                    table.shape[0], pairs.data_ptr(), _code(pairs), pairs.shape[0] - 1, int(mul_prev), int(mul_cur),
                                    last_token.data_ptr(), out.data_ptr(), copies, width, _stream()))
    return out


def stream_step(x: torch.Tensor, h: Optional[torch.Tensor] = None, y: Optional[torch.Tensor] = None,
                mix: Optional[torch.Tensor] = None, gain: Optional[torch.Tensor] = None, take: Optional[torch.Tensor] = None,
                weight: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None, eps: float = 0.0,
                centred: bool = True, rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """One pass over the streams ``x`` [streams, tokens, width] (32-bit), in up to three parts.  With ``y``: every
    stream becomes a mix of the old ones plus its share of y, x_t <- sum_s mix[s, t] x_s + gain[t] y, in place.  With
    ``h``: u = sum_t take[t] x_t (``take`` None: the plain sum) goes to ``h``, normed if ``weight`` is given:
    (u - mean) / sqrt(var + eps) * weight + bias, or without the mean if not ``centred``.  ``rows`` (int32): output
    row r reads row rows[r] (not with ``y``).  mix, gain and take are 32-bit."""
    _dev(x, "x")
    if x.dim() != 3 or x.dtype != torch.float32:
        raise KernelError(f"stream_step: x must be float32 [streams, tokens, width], got {x.dtype} {tuple(x.shape)}")
    streams, tokens, width = x.shape
    for t, what, count in ((mix, "mix", streams * streams), (gain, "gain", streams), (take, "take", streams)):
        if t is not None:
            _dev(t, what)
            if t.dtype != torch.float32 or t.numel() != count:
                raise KernelError(f"stream_step: {what} must be float32 with {count} entries")
    if y is not None:
        _dev(y, "y")
        if tuple(y.shape) != (tokens, width) or mix is None or gain is None or rows is not None:
            raise KernelError("stream_step: an update takes y [tokens, width], mix and gain, and no row list")
    out_rows = tokens
    if rows is not None:
        _dev(rows, "rows")
        if rows.dtype != torch.int32:
            raise KernelError("stream_step: rows must be int32")
        out_rows = rows.numel()
    if h is not None:
        _dev(h, "h")
        if tuple(h.shape) != (out_rows, width):
            raise KernelError(f"stream_step: h {tuple(h.shape)} against {out_rows} rows of {width}")
    if weight is not None:
        _dev(weight, "weight")
        if weight.numel() != width or (bias is not None and (bias.numel() != width or bias.dtype != weight.dtype)):
            raise KernelError("stream_step: the norm's weight and bias must have one entry per channel and one type")
    lib = core()
    _check(lib, lib.nnis_stream_step(x.data_ptr(), streams, tokens, width, _ptr(y), _code(y) if y is not None else 0, _ptr(mix),
                                     _ptr(gain), _ptr(take), _ptr(weight), _ptr(bias), _code(weight) if weight is not None else 0,
                                     1 if centred else 0, float(eps), _ptr(h), _code(h) if h is not None else 0, _ptr(rows),
                                     out_rows, _stream()))
    return h


def branch_mean(branches, weights, biases, eps: float, out: torch.Tensor) -> torch.Tensor:
    """out = mean over the branches of (y + b) / sqrt(mean((y + b)^2) + eps) * w: up to four inputs [tokens, width]
    of one type, each with a weight and a bias or None."""
    count = len(branches)
    if not 1 <= count <= 4 or len(weights) != count or len(biases) != count:
        raise KernelError("branch_mean: one to four branches, each with a weight and a bias or None")
    _dev(out, "out")
    tokens, width = out.shape
    for y, w, b in zip(branches, weights, biases):
        _dev(y, "branch"), _dev(w, "weight")
        if tuple(y.shape) != (tokens, width) or y.dtype != branches[0].dtype or w.numel() != width or w.dtype != weights[0].dtype:
            raise KernelError("branch_mean: branches and weights must agree in shape and type")
        if b is not None:
            _dev(b, "bias")
            if b.numel() != width or b.dtype != weights[0].dtype:
                raise KernelError("branch_mean: a bias has the weights' shape and type")
    pointers = lambda items: (ctypes.c_void_p * count)(*[None if t is None else t.data_ptr() for t in items])  # noqa: E731
    ys, ws, bs = pointers(branches), pointers(weights), pointers(biases)
    lib = core()
    _check(lib, lib.nnis_branch_mean(ctypes.cast(ys, _VOID), ctypes.cast(ws, _VOID), ctypes.cast(bs, _VOID), count,
                                     _code(branches[0]), _code(weights[0]), tokens, width, float(eps), out.data_ptr(), _code(out),
                                     _stream()))
    return out


ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "relu": 2}


def gated_act(gate_up: torch.Tensor, out: torch.Tensor, activation: str) -> torch.Tensor:
    """out = act(gate) * up on a fused [tokens, 2 * inner] projection, gate columns first."""
    if activation == "silu":
        return silu_mul(gate_up, out)
    _dev(gate_up, "gate_up"), _dev(out, "out")
    tokens, inner = out.shape
    if gate_up.shape != (tokens, 2 * inner) or activation not in ACTIVATIONS:
        raise KernelError(f"gated_act: gate_up {tuple(gate_up.shape)} against out {tuple(out.shape)}, activation {activation!r}")
    lib = core()
    _check(lib, lib.nnis_gated_act(gate_up.data_ptr(), _code(gate_up), out.data_ptr(), _code(out), tokens, inner,
                                   ACTIVATIONS[activation], _stream()))
    return out


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    _dev(y, "y"), _dev(bias, "bias")
    if y.dim() != 2 or bias.numel() != y.shape[1]:
        raise KernelError(f"add_bias: a bias of {bias.numel()} for rows of {tuple(y.shape)}")
    lib = core()
    _check(lib, lib.nnis_add_bias(y.data_ptr(), _code(y), bias.data_ptr(), _code(bias), y.shape[0], y.shape[1], _stream()))
    return y


# ---------------------------------------------------------------------------
# mixers that carry state
# ---------------------------------------------------------------------------

# A run of a sequence's tokens through a recurrence is a chain as long as the run; from RUN_PIECE_FROM tokens on the
# kernels cut it into pieces that run side by side (three passes, see csrc/recurrent.hip).  A piece has at least
# RUN_PIECE_LEAST tokens; the pieces' states between the passes take at most RUN_SCRATCH_BYTES.
RUN_PIECE_FROM = 48
RUN_PIECE_LEAST = 16
RUN_SCRATCH_BYTES = 256 << 20


def run_pieces(ctx, state_bytes: int):
    """(tokens of a piece, most pieces of a sequence) for a step whose longest run has ``ctx.max_new`` tokens, where a
    sequence's state takes ``state_bytes``; (0, 1) for a step that is not cut."""
    longest = int(ctx.max_new)
    if longest < RUN_PIECE_FROM:
        return 0, 1
    most = max(1, min(64, RUN_SCRATCH_BYTES // max(1, ctx.batch * state_bytes)))
    piece = max(RUN_PIECE_LEAST, -(-longest // most))
    pieces = -(-longest // piece)
    return (piece, pieces) if pieces > 1 else (0, 1)


def _step_arrays(ctx, what: str):
    for t in (ctx.tok_slot, ctx.tok_pos, ctx.seq_slot, ctx.seq_start):
        _dev(t, "step metadata")
        if t.dtype != torch.int32:
            raise KernelError(f"{what}: step metadata must be int32")
    if ctx.seq_start.numel() < ctx.batch + 1 or ctx.seq_slot.numel() < ctx.batch:
        raise KernelError(f"{what}: the step's sequence arrays are shorter than its {ctx.batch} sequences")


def conv_silu(x: torch.Tensor, channels: int, weight: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor],
              ctx, out: torch.Tensor) -> torch.Tensor:
    """out[t, c] = silu(bias[c] + sum_j weight[c, j] x[t - (taps - 1) + j, c]) over each sequence's own tokens, the
    last tap on the token itself.  ``x``: [tokens, >= channels], its first ``channels`` columns are taken.
    ``state`` (float32 [slots, taps - 1, channels]) holds each sequence's last inputs and is brought up to date."""
    _dev(x, "x"), _dev(weight, "weight"), _dev(out, "out")
    tokens = x.shape[0]
    taps = weight.shape[1]
    if weight.shape[0] != channels or x.shape[1] < channels or tuple(out.shape) != (tokens, channels):
        raise KernelError(f"conv_silu: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)} do not fit {channels} channels")
    if bias is not None and (bias.numel() != channels or bias.dtype != weight.dtype):
        raise KernelError("conv_silu: the bias has one entry per channel and the weight's type")
    if taps > 1:
        _dev(state, "state")
        if state.dtype != torch.float32 or tuple(state.shape[1:]) != (taps - 1, channels):
            raise KernelError(f"conv_silu: state must be float32 [slots, {taps - 1}, {channels}], got {tuple(state.shape)}")
    _step_arrays(ctx, "conv_silu")
    lib = recurrent()
    _check(lib, lib.nnis_conv_silu(x.data_ptr(), _code(x), x.stride(0), weight.data_ptr(), _ptr(bias), _code(weight), _ptr(state),
                                   ctx.tok_slot.data_ptr(), ctx.tok_pos.data_ptr(), ctx.seq_slot.data_ptr(), ctx.seq_start.data_ptr(),
                                   tokens, ctx.batch, channels, taps, out.data_ptr(), _code(out),
                                   1 if (ctx.decode and tokens == ctx.batch) else 0, _stream()))
    return out


def selective_scan(x: torch.Tensor, dt_pre: torch.Tensor, bc: torch.Tensor, z: torch.Tensor, A: torch.Tensor, D: torch.Tensor,
                   dt_bias: torch.Tensor, state: torch.Tensor, ctx, out: torch.Tensor) -> torch.Tensor:
    """The diagonal recurrence of a selective scan over each sequence's tokens, from and into ``state`` (float32
    [slots, channels, states]): dt = softplus(dt_pre + dt_bias); S <- exp(dt A) S + dt x B; out = (S . C + D x) *
    silu(z).  ``x`` [tokens, channels]; ``dt_pre`` float32 [tokens, channels]; ``bc`` float32 [tokens, 2 * states], B
    then C; ``z``: a view [tokens, channels] whose rows may be further apart; A, D, dt_bias float32."""
    tokens, channels = x.shape
    states = A.shape[1]
    for t, what in ((x, "x"), (dt_pre, "dt_pre"), (bc, "bc"), (A, "A"), (D, "D"), (dt_bias, "dt_bias"), (state, "state"), (out, "out")):
        _dev(t, what)
    for t, what, shape in ((dt_pre, "dt_pre", (tokens, channels)), (bc, "bc", (tokens, 2 * states)), (A, "A", (channels, states)),
                           (D, "D", (channels,)), (dt_bias, "dt_bias", (channels,))):
        if t.dtype != torch.float32 or tuple(t.shape) != shape:
            raise KernelError(f"selective_scan: {what} must be float32 {shape}, got {t.dtype} {tuple(t.shape)}")
    if state.dtype != torch.float32 or tuple(state.shape[1:]) != (channels, states) or tuple(out.shape) != (tokens, channels):
        raise KernelError("selective_scan: state must be float32 [slots, channels, states] and out [tokens, channels]")
    if not z.is_cuda or tuple(z.shape) != (tokens, channels) or z.stride(1) != 1:
        raise KernelError("selective_scan: z must be [tokens, channels] on the GPU with adjacent columns")
    _step_arrays(ctx, "selective_scan")
    piece, pieces = run_pieces(ctx, channels * states * 4)
    carried = stepped = None
    if pieces > 1:
        carried = torch.empty(ctx.batch * pieces * channels * states, dtype=torch.float32, device=x.device)
        stepped = torch.empty(ctx.batch * pieces * channels, dtype=torch.float32, device=x.device)
    lib = recurrent()
    _check(lib, lib.nnis_selective_scan(x.data_ptr(), _code(x), dt_pre.data_ptr(), bc.data_ptr(), z.data_ptr(), _code(z),
                                        z.stride(0) if tokens > 1 else channels, A.data_ptr(), D.data_ptr(), dt_bias.data_ptr(),
                                        state.data_ptr(), ctx.seq_slot.data_ptr(), ctx.seq_start.data_ptr(), ctx.batch, channels,
                                        states, out.data_ptr(), _code(out), piece, pieces, _ptr(carried), _ptr(stepped), _stream()))
    return out


def gla_decays(logits: torch.Tensor, bias: torch.Tensor, tau: float) -> torch.Tensor:
    """In place: logits <- log(sigmoid(logits + bias)) / tau, the logarithms of the decays sigmoid(.)^(1 / tau) that
    ``gla_scan`` takes.  Both float32; ``bias`` has one entry per column."""
    _dev(logits, "logits"), _dev(bias, "bias")
    if logits.dtype != torch.float32 or bias.dtype != torch.float32 or logits.dim() != 2 or bias.numel() != logits.shape[1]:
        raise KernelError("gla_decays: logits must be float32 [tokens, channels] and the bias float32 [channels]")
    lib = recurrent()
    _check(lib, lib.nnis_gla_decays(logits.data_ptr(), bias.data_ptr(), logits.shape[0], logits.shape[1], float(tau), _stream()))
    return logits


def gla_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay_logs: Optional[torch.Tensor], scale: float,
             state: torch.Tensor, ctx, heads: int, out: torch.Tensor, head_decay: Optional[torch.Tensor] = None,
             rotation=None) -> torch.Tensor:
    """Gated linear attention over each sequence's tokens, from and into ``state`` (float32 [slots, heads, key
    channels, value channels]): alpha = exp(decay_logs); S <- diag(alpha) S + k v^T; out = S^T (q * scale), raw,
    float32 [tokens, heads * value channels].  q, k [tokens, heads * key channels] and v are views whose rows may be
    further apart; ``decay_logs`` float32 [tokens, heads * key channels] (``gla_decays``).  Without ``decay_logs``:
    ``head_decay`` float32 [2, heads], one fixed decay a head and its logarithm (retention).  ``rotation``: (cos, sin,
    rot_dim): the first rot_dim channels of every head of q and k are turned by the token's position while the kernel
    stages them, channel i with channel i + rot_dim / 2, in 32-bit (tables float32 [positions, rot_dim / 2])."""
    decay_logits = decay_logs
    tokens = q.shape[0]
    key_dim, value_dim = q.shape[1] // heads, v.shape[1] // heads
    for t, what in ((q, "q"), (k, "k"), (v, "v")):
        if not t.is_cuda or t.stride(1) != 1 or t.dtype != q.dtype or t.shape[0] != tokens:
            raise KernelError(f"gla_scan: {what} must be [tokens, channels] on the GPU with adjacent columns, of one type")
    if k.shape[1] != heads * key_dim or q.shape[1] != heads * key_dim or v.shape[1] != heads * value_dim:
        raise KernelError(f"gla_scan: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)} do not fit {heads} heads")
    _dev(state, "state"), _dev(out, "out")
    if (decay_logits is None) == (head_decay is None):
        raise KernelError("gla_scan: decays a token and channel, or one a head")
    if decay_logits is not None:
        _dev(decay_logits, "decay_logits")
        if decay_logits.dtype != torch.float32 or tuple(decay_logits.shape) != (tokens, heads * key_dim):
            raise KernelError("gla_scan: decay_logits must be float32 [tokens, heads * key channels]")
    else:
        _dev(head_decay, "head_decay")
        if head_decay.dtype != torch.float32 or tuple(head_decay.shape) != (2, heads) or not head_decay.is_contiguous():
            raise KernelError(f"gla_scan: head_decay must be float32 [2, {heads}], got {tuple(head_decay.shape)}")
    cos = sin = None
    rot_dim = 0
    if rotation is not None:
        cos, sin, rot_dim = rotation
        _dev(cos, "cos"), _dev(sin, "sin")
        if (cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2
                or cos.shape[1] != rot_dim // 2 or rot_dim % 2 or rot_dim > key_dim or ctx.tok_pos.numel() < tokens):
            raise KernelError(f"gla_scan: tables {tuple(cos.shape)} do not fit a rotation of {rot_dim} channels in heads of {key_dim}")
    if state.dtype != torch.float32 or tuple(state.shape[1:]) != (heads, key_dim, value_dim):
        raise KernelError(f"gla_scan: state must be float32 [slots, {heads}, {key_dim}, {value_dim}], got {tuple(state.shape)}")
    if out.dtype != torch.float32 or tuple(out.shape) != (tokens, heads * value_dim):
        raise KernelError("gla_scan: out must be float32 [tokens, heads * value channels]")
    _step_arrays(ctx, "gla_scan")
    stride = lambda t: t.stride(0) if tokens > 1 else t.shape[1]  # noqa: E731
    piece, pieces = run_pieces(ctx, heads * key_dim * value_dim * 4)
    carried = decayed = None
    if pieces > 1:
        carried = torch.empty(ctx.batch * pieces * heads * key_dim * value_dim, dtype=torch.float32, device=out.device)
        decayed = torch.empty(ctx.batch * pieces * heads * key_dim, dtype=torch.float32, device=out.device)
    lib = recurrent()
    _check(lib, lib.nnis_gla_scan_turned(q.data_ptr(), k.data_ptr(), v.data_ptr(), _code(q), stride(q), stride(k), stride(v),
                                         _ptr(decay_logits), _ptr(head_decay), _ptr(cos), _ptr(sin), rot_dim,
                                         cos.shape[0] if cos is not None else 0, ctx.tok_pos.data_ptr(), float(scale),
                                         state.data_ptr(), ctx.seq_slot.data_ptr(), ctx.seq_start.data_ptr(), ctx.batch, heads,
                                         key_dim, value_dim, out.data_ptr(), piece, pieces, _ptr(carried), _ptr(decayed), _stream()))
    return out


def head_norm_gate(o: torch.Tensor, gate: torch.Tensor, weight: Optional[torch.Tensor], eps: float, heads: int, out: torch.Tensor) -> torch.Tensor:
    """out[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * weight * silu(gate[t, h, :]); ``o`` float32
    [tokens, heads * dim], ``gate`` a view of that shape whose rows may be further apart, ``weight`` [dim] or None
    (a norm without a weight)."""
    _dev(o, "o"), _dev(out, "out")
    tokens = o.shape[0]
    dim = o.shape[1] // heads
    if weight is not None:
        _dev(weight, "weight")
    if o.dtype != torch.float32 or o.shape[1] != heads * dim or (weight is not None and weight.numel() != dim) or tuple(out.shape) != tuple(o.shape):
        raise KernelError(f"head_norm_gate: o {tuple(o.shape)}, weight, out {tuple(out.shape)} do not fit {heads} heads")
    if not gate.is_cuda or tuple(gate.shape) != tuple(o.shape) or gate.stride(1) != 1:
        raise KernelError("head_norm_gate: the gate must be [tokens, heads * dim] on the GPU with adjacent columns")
    lib = recurrent()
    _check(lib, lib.nnis_head_norm_gate(o.data_ptr(), gate.data_ptr(), _code(gate), gate.stride(0) if tokens > 1 else gate.shape[1],
                                        _ptr(weight), _code(weight) if weight is not None else 0, out.data_ptr(), _code(out), tokens,
                                        heads, dim, float(eps), _stream()))
    return out


def gated_delta(rows: torch.Tensor, ba: torch.Tensor, rate: torch.Tensor, dt_bias: torch.Tensor, q_scale: float, state: torch.Tensor,
                ctx, heads: int, groups: int, key_dim: int, value_dim: int, out: torch.Tensor, unit_eps: float = 1e-6) -> torch.Tensor:
    """The gated delta rule over each sequence's tokens, from and into ``state`` (float32 [slots, heads, value channels,
    key channels]: S column by column): S <- g S; u = beta (v - S^T k); S <- S + k u^T; out = S^T q, raw, float32 [tokens, heads * value
    channels].  ``rows`` [tokens, >= 2 * groups * key_dim + heads * value_dim]: q and k of ``groups`` heads, then v; q
    and k are made unit vectors per head (x / sqrt(sum x^2 + unit_eps)), q also times ``q_scale``.  ``ba`` float32
    [tokens, 2 * heads]: beta = sigmoid(first half), g = exp(-rate * softplus(second half + dt_bias)); ``rate`` and
    ``dt_bias`` float32 [heads]."""
    _dev(rows, "rows"), _dev(ba, "ba"), _dev(rate, "rate"), _dev(dt_bias, "dt_bias"), _dev(state, "state"), _dev(out, "out")
    tokens = rows.shape[0]
    if rows.dim() != 2 or rows.stride(1) != 1 or rows.shape[1] < 2 * groups * key_dim + heads * value_dim:
        raise KernelError(f"gated_delta: rows {tuple(rows.shape)} do not hold {groups} query/key heads of {key_dim} and {heads} values of {value_dim}")
    if ba.dtype != torch.float32 or tuple(ba.shape) != (tokens, 2 * heads) or not ba.is_contiguous():
        raise KernelError(f"gated_delta: ba must be float32 [tokens, {2 * heads}], got {tuple(ba.shape)}")
    for t, what in ((rate, "rate"), (dt_bias, "dt_bias")):
        if t.dtype != torch.float32 or t.numel() != heads:
            raise KernelError(f"gated_delta: {what} must be float32 [{heads}]")
    if state.dtype != torch.float32 or tuple(state.shape[1:]) != (heads, value_dim, key_dim):
        raise KernelError(f"gated_delta: state must be float32 [slots, {heads}, {value_dim}, {key_dim}], got {tuple(state.shape)}")
    if out.dtype != torch.float32 or tuple(out.shape) != (tokens, heads * value_dim):
        raise KernelError("gated_delta: out must be float32 [tokens, heads * value channels]")
    _step_arrays(ctx, "gated_delta")
    # between the two kernels: the unit vectors, g and beta, and the products q . k, all 32-bit
    scratch = torch.empty(max(1, tokens * (groups * 2 * key_dim + 2 * heads + groups)), dtype=torch.float32, device=out.device)
    lib = recurrent()
    _check(lib, lib.nnis_gated_delta(rows.data_ptr(), _code(rows), rows.stride(0) if tokens > 1 else rows.shape[1], ba.data_ptr(),
                                     rate.data_ptr(), dt_bias.data_ptr(), float(q_scale), float(unit_eps), state.data_ptr(),
                                     ctx.seq_slot.data_ptr(), ctx.seq_start.data_ptr(), ctx.batch, tokens, heads, groups, key_dim,
                                     value_dim, out.data_ptr(), scratch.data_ptr(), _stream()))
    return out


def branch_sum(branches, scales, out: torch.Tensor) -> torch.Tensor:
    """out = sum over the branches of scale * y: up to four inputs of one type and of out's shape, the sum in 32-bit."""
    count = len(branches)
    if not 1 <= count <= 4 or len(scales) != count:
        raise KernelError("branch_sum: one to four branches, each with a factor")
    _dev(out, "out")
    for y in branches:
        _dev(y, "branch")
        if y.shape != out.shape or y.dtype != branches[0].dtype or not y.is_contiguous():
            raise KernelError("branch_sum: branches must agree with the output in shape and with one another in type")
    ys = (ctypes.c_void_p * count)(*[y.data_ptr() for y in branches])
    factors = (ctypes.c_float * count)(*[float(value) for value in scales])
    lib = core()
    _check(lib, lib.nnis_branch_sum(ctypes.cast(ys, _VOID), ctypes.cast(factors, _VOID), count, _code(branches[0]), out.numel(),
                                    out.data_ptr(), _code(out), _stream()))
    return out


def scale_rows(x: torch.Tensor, factor: float) -> torch.Tensor:
    """x *= factor, in place, on 32-bit rows."""
    _dev(x, "x")
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError(f"scale_rows: 32-bit rows are needed, got {x.dtype}")
    lib = core()
    _check(lib, lib.nnis_scale_rows(x.data_ptr(), float(factor), x.numel(), _stream()))
    return x


# ---------------------------------------------------------------------------
# the residual's step around a norm without statistics; logits bent by a cap
# ---------------------------------------------------------------------------

def tanh_norm_step(x: Optional[torch.Tensor], x_out: Optional[torch.Tensor] = None, y: Optional[torch.Tensor] = None, post=None,
                   rows_add: Optional[torch.Tensor] = None, vec_add: Optional[torch.Tensor] = None, following=None,
                   h: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """One kernel for what lies between two projections of a layer whose
    norm is y -> tanh(alpha y) w + b.  ``x``: the 32-bit stream [tokens,
    width], or None for a stream of zeros (then ``y`` gives the shape).  v = x + (``post`` ? post(y) : y) + rows_add + vec_add, each term
    only if given; ``x_out`` (x itself, or another tensor of its shape) takes
    v; ``h`` takes ``following``(v), or v without one.  ``post`` /
    ``following``: (alpha, weight, bias).  ``rows`` (int32): output row r
    reads row rows[r]; the stream is then left as it is.  Returns ``h``."""
    shape_of = x if x is not None else y
    if shape_of is None or shape_of.dim() != 2:
        raise KernelError("tanh_norm_step: a stream or an output [tokens, width] is needed")
    if x is not None:
        _dev(x, "x")
        if x.dtype != torch.float32:
            raise KernelError(f"tanh_norm_step: the stream is float32, got {x.dtype}")
    tokens, width = shape_of.shape
    out_rows = tokens
    if rows is not None:
        _dev(rows, "rows")
        if rows.dtype != torch.int32:
            raise KernelError("tanh_norm_step: rows must be int32")
        out_rows = rows.numel()
        if x_out is not None:
            raise KernelError("tanh_norm_step: a step over a list of rows leaves the stream as it is")
    for t, what in ((x_out, "x_out"), (rows_add, "rows_add")):
        if t is not None:
            _dev(t, what)
            if t.dtype != torch.float32 or t.shape != shape_of.shape:
                raise KernelError(f"tanh_norm_step: {what} {tuple(t.shape)} {t.dtype} against the stream {tuple(shape_of.shape)}")
    if y is not None:
        _dev(y, "y")
        if y.shape != shape_of.shape:
            raise KernelError(f"tanh_norm_step: y {tuple(y.shape)} against the stream {tuple(shape_of.shape)}")
    w_code = None
    for norm, what in ((post, "post"), (following, "following")):
        if norm is not None:
            _, weight, bias = norm
            _dev(weight, f"{what} weight"), _dev(bias, f"{what} bias")
            if weight.numel() != width or bias.numel() != width or weight.dtype != bias.dtype:
                raise KernelError(f"tanh_norm_step: the {what} norm's weight and bias do not fit a width of {width}")
            if w_code is not None and _code(weight) != w_code:
                raise KernelError("tanh_norm_step: the norms' weights differ in type")
            w_code = _code(weight)
    if vec_add is not None:
        _dev(vec_add, "vec_add")
        if vec_add.numel() != width or (w_code is not None and _code(vec_add) != w_code):
            raise KernelError(f"tanh_norm_step: the vector does not fit a width of {width} or the weights' type")
        w_code = _code(vec_add)
    if post is not None and y is None:
        raise KernelError("tanh_norm_step: a norm on the way in needs something to norm")
    if h is not None:
        _dev(h, "h")
        if h.shape != (out_rows, width):
            raise KernelError(f"tanh_norm_step: h {tuple(h.shape)} against {out_rows} rows of {width}")
    lib = core()
    _check(lib, lib.nnis_tanh_norm_step(
        _ptr(x), _ptr(x_out), _ptr(y), _code(y) if y is not None else 0,
        _ptr(post[1]) if post else None, _ptr(post[2]) if post else None, float(post[0]) if post else 0.0,
        _ptr(rows_add), _ptr(vec_add), _ptr(following[1]) if following else None, _ptr(following[2]) if following else None,
        float(following[0]) if following else 0.0, w_code or 0, _ptr(h), _code(h) if h is not None else 0, _ptr(rows),
        out_rows, width, _stream()))
    return h


def tanh_cap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x -> cap * tanh(x / cap), in place, on 32-bit rows."""
    _dev(x, "x")
    if x.dtype != torch.float32 or not cap > 0.0:
        raise KernelError(f"tanh_cap: 32-bit rows and a positive cap are needed, got {x.dtype} and {cap}")
    lib = core()
    _check(lib, lib.nnis_tanh_cap(x.data_ptr(), float(cap), x.numel(), _stream()))
    return x


# ---------------------------------------------------------------------------
# attention over a cached latent: between the projections
# ---------------------------------------------------------------------------

def latent_prepare(proj: torch.Tensor, q_rank: int, kv_rank: int, rot_dim: int, gates: int, q_weight: Optional[torch.Tensor],
                   c_weight: torch.Tensor, eps: float, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                   tok_slot: torch.Tensor, tok_pos: torch.Tensor, cq: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                   v_pages: Optional[torch.Tensor], block_table: Optional[torch.Tensor], gate: Optional[torch.Tensor]) -> None:
    """From the rows of one fused projection, [query latent (q_rank) | latent
    (kv_rank) | rotated key part (rot_dim) | gate logits (gates)]: ``cq`` takes
    the query latent over its root mean square times ``q_weight``; the latent
    likewise with ``c_weight``, written as the first kv_rank key channels and
    as the value of each token's place in the pages (one key/value head, keys
    of kv_rank + rot_dim channels, values of kv_rank), the rotated key part
    (pairs of neighbouring channels turned by the token's position) behind it
    in the keys; ``gate`` (float32) takes sigmoid of the gate logits."""
    _dev(proj, "proj"), _dev(c_weight, "c_weight"), _dev(tok_slot, "tok_slot"), _dev(tok_pos, "tok_pos")
    tokens = proj.shape[0]
    if proj.dim() != 2 or proj.shape[1] != q_rank + kv_rank + rot_dim + gates:
        raise KernelError(f"latent_prepare: rows of {proj.shape[1]} against {q_rank} + {kv_rank} + {rot_dim} + {gates}")
    if c_weight.numel() != kv_rank or (q_rank and (q_weight is None or q_weight.numel() != q_rank or q_weight.dtype != c_weight.dtype)):
        raise KernelError("latent_prepare: the norms' weights do not fit the latents")
    if tok_slot.dtype != torch.int32 or tok_pos.dtype != torch.int32 or min(tok_slot.numel(), tok_pos.numel()) < tokens:
        raise KernelError("latent_prepare: tok_slot / tok_pos must be int32 with one entry per token")
    if q_rank:
        _dev(cq, "cq")
        if cq.shape != (tokens, q_rank):
            raise KernelError(f"latent_prepare: cq {tuple(cq.shape)} against {tokens} rows of {q_rank}")
    positions = 0
    if rot_dim:
        _dev(cos, "cos"), _dev(sin, "sin")
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[1] != rot_dim // 2:
            raise KernelError(f"latent_prepare: tables {tuple(cos.shape)} do not fit rot_dim {rot_dim} in float32")
        positions = cos.shape[0]
    if gates:
        _dev(gate, "gate")
        if gate.dtype != torch.float32 or gate.shape != (tokens, gates):
            raise KernelError(f"latent_prepare: gate must be float32 [{tokens}, {gates}]")
    max_pages = cache_code = 0
    if k_pages is not None:
        _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(block_table, "block_table")
        if not _pages_fit(k_pages, v_pages, 1, kv_rank + rot_dim, kv_rank) or k_pages.dtype != v_pages.dtype:
            raise KernelError(f"latent_prepare: page shapes {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not fit")
        if block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise KernelError("latent_prepare: block_table must be int32 [slots, pages]")
        max_pages, cache_code = block_table.shape[1], _code(k_pages)
    lib = latent()
    _check(lib, lib.nnis_latent_prepare(proj.data_ptr(), _code(proj), tokens, q_rank, kv_rank, rot_dim, gates, _ptr(q_weight),
                                        c_weight.data_ptr(), _code(c_weight), float(eps), _ptr(cos), _ptr(sin), positions,
                                        tok_slot.data_ptr(), tok_pos.data_ptr(), _ptr(cq), _code(cq) if cq is not None else 0,
                                        _ptr(k_pages), _ptr(v_pages), cache_code, _ptr(block_table), max_pages, _ptr(gate), _stream()))


def latent_rotate_q(q: torch.Tensor, heads: int, head_width: int, first: int, rot_dim: int, cos: torch.Tensor, sin: torch.Tensor,
                    tok_pos: torch.Tensor) -> torch.Tensor:
    """Turns channels [first, first + rot_dim) of every head of ``q`` [tokens,
    heads * head_width] by each token's position, pairs of neighbouring
    channels, in place."""
    _dev(q, "q"), _dev(cos, "cos"), _dev(sin, "sin"), _dev(tok_pos, "tok_pos")
    tokens = q.shape[0]
    if q.shape != (tokens, heads * head_width) or tok_pos.dtype != torch.int32 or tok_pos.numel() < tokens:
        raise KernelError(f"latent_rotate_q: q {tuple(q.shape)} against {heads} heads of {head_width}")
    if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[1] != rot_dim // 2:
        raise KernelError(f"latent_rotate_q: tables {tuple(cos.shape)} do not fit rot_dim {rot_dim} in float32")
    lib = latent()
    _check(lib, lib.nnis_latent_rotate_q(q.data_ptr(), _code(q), tokens, heads, head_width, first, rot_dim, cos.data_ptr(),
                                         sin.data_ptr(), cos.shape[0], tok_pos.data_ptr(), _stream()))
    return q


def head_scale(o: torch.Tensor, gate: torch.Tensor, heads: int, logistic: bool = False) -> torch.Tensor:
    """o[t, h, :] *= gate[t, h], in place; ``o`` [tokens, heads * channels], ``gate`` float32 [tokens, heads].
    ``logistic``: the gates are logits still, and the factor is sigmoid(gate[t, h])."""
    _dev(o, "o"), _dev(gate, "gate")
    tokens = o.shape[0]
    if o.shape[1] % heads or gate.shape != (tokens, heads) or gate.dtype != torch.float32:
        raise KernelError(f"head_scale: o {tuple(o.shape)} and gate {tuple(gate.shape)} {gate.dtype} do not fit {heads} heads")
    lib = latent()
    if not gate.is_contiguous() or not o.is_contiguous():
        raise KernelError("head_scale: rows and gates lie one behind the other")
    _check(lib, lib.nnis_head_scale_of(o.data_ptr(), _code(o), gate.data_ptr(), tokens, heads, o.shape[1] // heads,
                                       1 if logistic else 0, _stream()))
    return o


def heads_linear(x: torch.Tensor, weight: torch.Tensor, gate: Optional[torch.Tensor], heads: int, out: torch.Tensor) -> torch.Tensor:
    """out[t, h, :] = (weight[h] @ x[t, h, :]) * gate[t, h, :]: a map of its own for every head.  ``x`` [tokens, heads *
    K], ``weight`` [heads, N, K], ``gate`` float32 [tokens, heads * N] or None, ``out`` [tokens, heads * N]."""
    _dev(x, "x"), _dev(weight, "weight"), _dev(out, "out")
    tokens = x.shape[0]
    if weight.dim() != 3 or weight.shape[0] != heads or not weight.is_contiguous() or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"heads_linear: a weight [heads, N, K] is needed, got {tuple(weight.shape)}")
    n, k = weight.shape[1], weight.shape[2]
    if tuple(x.shape) != (tokens, heads * k) or tuple(out.shape) != (tokens, heads * n):
        raise KernelError(f"heads_linear: x {tuple(x.shape)} and out {tuple(out.shape)} against {heads} maps of {n} x {k}")
    if gate is not None:
        _dev(gate, "gate")
        if gate.dtype != torch.float32 or tuple(gate.shape) != (tokens, heads * n) or not gate.is_contiguous():
            raise KernelError(f"heads_linear: the gate must be float32 [tokens, {heads * n}], got {tuple(gate.shape)}")
    lib = latent()
    _check(lib, lib.nnis_heads_linear(x.data_ptr(), _code(x), weight.data_ptr(), _code(weight), _ptr(gate), out.data_ptr(), _code(out),
                                      tokens, heads, n, k, _stream()))
    return out


# ---------------------------------------------------------------------------
# sublayers that norm their outputs, gate or pool their heads, or route their tokens
# ---------------------------------------------------------------------------

def cast_rows(x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[r] = x[rows[r]] (or x[r] without ``rows``) in out's type."""
    _dev(x, "x"), _dev(out, "out")
    if x.dim() != 2 or out.dim() != 2 or out.shape[1] != x.shape[1] or (rows is None and out.shape[0] != x.shape[0]):
        raise KernelError(f"cast_rows: x {tuple(x.shape)} against out {tuple(out.shape)}")
    if rows is not None:
        _dev(rows, "rows")
        if rows.dtype != torch.int32 or rows.numel() < out.shape[0]:
            raise KernelError("cast_rows: rows must be int32 with one entry per output row")
    lib = sublayer()
    _check(lib, lib.nnis_cast_rows(x.data_ptr(), _code(x), out.data_ptr(), _code(out), _ptr(rows), out.shape[0], x.shape[1], _stream()))
    return out


def rms_post_step(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, offset: float, eps: float,
                  h: Optional[torch.Tensor] = None, share=None) -> Optional[torch.Tensor]:
    """x += y / sqrt(mean(y^2) + eps) * (offset + weight), row by row, in place in the 32-bit stream ``x``; ``h`` (of
    x's shape, any type) receives the new rows.  ``share``: (keep float32 [rows], rows of x's shape): y then stands
    for y + keep[row] * rows[row]; the rows may be ``h`` or ``x`` themselves."""
    _dev(x, "x"), _dev(y, "y"), _dev(weight, "norm weight")
    if x.dtype != torch.float32 or x.dim() != 2 or y.shape != x.shape or weight.numel() != x.shape[1]:
        raise KernelError(f"rms_post_step: a float32 stream {tuple(x.shape)} against y {tuple(y.shape)} and a weight of {weight.numel()}")
    if h is not None:
        _dev(h, "h")
        if h.shape != x.shape:
            raise KernelError(f"rms_post_step: h {tuple(h.shape)} against the stream {tuple(x.shape)}")
    lib = sublayer()
    keep = rows_in = None
    if share is not None:
        keep, rows_in = share
        _dev(keep, "keep"), _dev(rows_in, "shared rows")
        if keep.dtype != torch.float32 or keep.numel() != x.shape[0] or rows_in.shape != x.shape or not rows_in.is_contiguous():
            raise KernelError(f"rms_post_step: a float32 share per row and rows {tuple(x.shape)}, got {tuple(keep.shape)} and {tuple(rows_in.shape)}")
    _check(lib, lib.nnis_rms_post_step(x.data_ptr(), y.data_ptr(), _code(y), weight.data_ptr(), _code(weight), float(offset), float(eps),
                                       _ptr(h), _code(h) if h is not None else 0, x.shape[0], x.shape[1], _ptr(keep), _ptr(rows_in),
                                       _code(rows_in) if rows_in is not None else 0, _stream()))
    return h


def rms_between(x: torch.Tensor, y: torch.Tensor, w_out: torch.Tensor, w_in: Optional[torch.Tensor], eps: float,
                h: Optional[torch.Tensor] = None, share=None) -> Optional[torch.Tensor]:
    """Between two sublayers that are normed both ways: x += y / sqrt(mean(y^2) + eps) * w_out, row by row, in place in
    the 32-bit stream ``x``, and h = x / sqrt(mean(x^2) + eps) * w_in (``h`` and ``w_in`` together, or neither).
    ``share`` as in ``rms_post_step``.  The two weights have one type."""
    _dev(x, "x"), _dev(y, "y"), _dev(w_out, "norm weight")
    if x.dtype != torch.float32 or x.dim() != 2 or y.shape != x.shape or w_out.numel() != x.shape[1] or not y.is_contiguous():
        raise KernelError(f"rms_between: a float32 stream {tuple(x.shape)} against y {tuple(y.shape)} and a weight of {w_out.numel()}")
    if (h is None) != (w_in is None):
        raise KernelError("rms_between: the rows out come with the next norm's weight")
    if h is not None:
        _dev(h, "h"), _dev(w_in, "next norm weight")
        if h.shape != x.shape or w_in.numel() != x.shape[1] or w_in.dtype != w_out.dtype:
            raise KernelError(f"rms_between: h {tuple(h.shape)} and the next weight against the stream {tuple(x.shape)}")
    keep = rows_in = None
    if share is not None:
        keep, rows_in = share
        _dev(keep, "keep"), _dev(rows_in, "shared rows")
        if keep.dtype != torch.float32 or keep.numel() != x.shape[0] or rows_in.shape != x.shape or not rows_in.is_contiguous():
            raise KernelError(f"rms_between: a float32 share per row and rows {tuple(x.shape)}, got {tuple(keep.shape)} and {tuple(rows_in.shape)}")
    lib = sublayer()
    _check(lib, lib.nnis_rms_between(x.data_ptr(), y.data_ptr(), _code(y), w_out.data_ptr(), _ptr(w_in), _code(w_out), float(eps), _ptr(h),
                                     _code(h) if h is not None else 0, x.shape[0], x.shape[1], _ptr(keep), _ptr(rows_in),
                                     _code(rows_in) if rows_in is not None else 0, _stream()))
    return h


def poly_norm(z: torch.Tensor, coefficients: torch.Tensor, eps: float, out: torch.Tensor) -> torch.Tensor:
    """out = a N(z) + b N(z^2) + c N(z^3) + e row by row, N(v) = v / sqrt(mean(v^2) + eps); ``coefficients``: float32
    (a, b, c, e) on the device."""
    _dev(z, "z"), _dev(coefficients, "coefficients"), _dev(out, "out")
    if z.dim() != 2 or out.shape != z.shape or coefficients.dtype != torch.float32 or coefficients.numel() != 4:
        raise KernelError(f"poly_norm: z {tuple(z.shape)}, out {tuple(out.shape)}, four float32 coefficients")
    lib = sublayer()
    _check(lib, lib.nnis_poly_norm(z.data_ptr(), _code(z), coefficients.data_ptr(), float(eps), out.data_ptr(), _code(out), z.shape[0],
                                   z.shape[1], _stream()))
    return out


ROUTE_MOST_OUTPUTS = 1024
ROUTE_MOST_CHANNELS = 16384


def router_logits(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[row, e] = x[row] . weight[e] in 32-bit: ``weight`` float32 [outputs, width], ``out`` float32 [rows, outputs];
    ``x`` in either type."""
    _dev(x, "x"), _dev(weight, "router weight"), _dev(out, "out")
    rows, width = x.shape
    if (x.dim() != 2 or not x.is_contiguous() or weight.dtype != torch.float32 or weight.dim() != 2 or weight.shape[1] != width
            or out.dtype != torch.float32 or tuple(out.shape) != (rows, weight.shape[0]) or width > ROUTE_MOST_CHANNELS):
        raise KernelError(f"router_logits: x {tuple(x.shape)}, a float32 weight {tuple(weight.shape)}, float32 out {tuple(out.shape)}")
    lib = sublayer()
    _check(lib, lib.nnis_router_logits(x.data_ptr(), _code(x), weight.data_ptr(), out.data_ptr(), rows, weight.shape[0], width, _stream()))
    return out


def _route_groups(groups, n: int, what: str):
    """(count, keep) of a router whose outputs form equal groups of neighbours, (1, 1) without."""
    if groups is None:
        return 1, 1
    count, keep = int(groups[0]), int(groups[1])
    if not (1 <= count <= 64 and n % count == 0 and 1 <= keep <= count):
        raise KernelError(f"{what}: {n} outputs in {count} equal groups (up to 64) of which {keep} are kept")
    return count, keep


def route_top(logits: torch.Tensor, correction: Optional[torch.Tensor], experts: int, top: int, gates: torch.Tensor,
              keep: torch.Tensor, groups=None):
    """Scores softmax(logits) [rows, n]; the ``top`` largest of score + correction are chosen.  ``gates`` [rows, experts]
    gets the score of every chosen output below ``experts`` and 0 elsewhere; ``keep`` [rows] the summed scores of the
    chosen outputs from ``experts`` on.  All float32."""
    _dev(logits, "logits"), _dev(gates, "gates"), _dev(keep, "keep")
    rows, n = logits.shape
    if logits.dtype != torch.float32 or gates.dtype != torch.float32 or keep.dtype != torch.float32 \
            or tuple(gates.shape) != (rows, experts) or keep.numel() != rows:
        raise KernelError(f"route_top: float32 logits {tuple(logits.shape)}, gates {tuple(gates.shape)}, keep {tuple(keep.shape)}")
    if correction is not None:
        _dev(correction, "correction")
        if correction.dtype != torch.float32 or correction.numel() != n:
            raise KernelError(f"route_top: a float32 correction per output ({n}), got {tuple(correction.shape)} {correction.dtype}")
    if not (0 < n <= ROUTE_MOST_OUTPUTS and 0 <= experts <= n and 0 < top <= n):
        raise KernelError(f"route_top: {experts} experts and the {top} largest of {n} outputs (at most {ROUTE_MOST_OUTPUTS})")
    group_count, group_keep = _route_groups(groups, n, "route_top")
    lib = sublayer()
    _check(lib, lib.nnis_route_top(logits.data_ptr(), _ptr(correction), rows, n, experts, top, gates.data_ptr(), keep.data_ptr(),
                                   group_count, group_keep, _stream()))
    return gates, keep


ROUTE_FUSED_MOST_CHANNELS = 8192


def route(x: torch.Tensor, weight: torch.Tensor, correction: Optional[torch.Tensor], experts: int, top: int, gates: torch.Tensor,
          keep: torch.Tensor, groups=None):
    """``router_logits`` and ``route_top`` in one kernel (rows of up to ``ROUTE_FUSED_MOST_CHANNELS`` channels).
    ``groups``: (count, keep): the outputs form ``count`` equal groups of neighbours, a group's mark is its largest
    corrected score, and only outputs of the ``keep`` groups with the largest marks can be chosen."""
    _dev(x, "x"), _dev(weight, "router weight"), _dev(gates, "gates"), _dev(keep, "keep")
    rows, width = x.shape
    n = weight.shape[0]
    if (x.dim() != 2 or not x.is_contiguous() or weight.dtype != torch.float32 or weight.dim() != 2 or weight.shape[1] != width
            or gates.dtype != torch.float32 or keep.dtype != torch.float32 or tuple(gates.shape) != (rows, experts) or keep.numel() != rows):
        raise KernelError(f"route: x {tuple(x.shape)}, a float32 weight {tuple(weight.shape)}, float32 gates {tuple(gates.shape)} and keep {tuple(keep.shape)}")
    if correction is not None:
        _dev(correction, "correction")
        if correction.dtype != torch.float32 or correction.numel() != n:
            raise KernelError(f"route: a float32 correction per output ({n}), got {tuple(correction.shape)} {correction.dtype}")
    if not (0 < n <= ROUTE_MOST_OUTPUTS and 0 <= experts <= n and 0 < top <= n and width <= ROUTE_FUSED_MOST_CHANNELS):
        raise KernelError(f"route: {experts} experts and the {top} largest of {n} outputs (at most {ROUTE_MOST_OUTPUTS}) of rows of {width} channels")
    group_count, group_keep = _route_groups(groups, n, "route")
    lib = sublayer()
    _check(lib, lib.nnis_route(x.data_ptr(), _code(x), weight.data_ptr(), _ptr(correction), rows, n, width, experts, top, gates.data_ptr(),
                               keep.data_ptr(), group_count, group_keep, _stream()))
    return gates, keep


def routed_act(z: torch.Tensor, gates: torch.Tensor, out: torch.Tensor, form: str = "relu_squared") -> torch.Tensor:
    """On the experts' fused up projection.  ``relu_squared``: out[row, e * ff + c] = gates[row, e] * relu(z[row, e * ff
    + c])^2.  ``silu_gated``: z [rows, experts * 2 * ff] holds, expert by expert, gate columns then up columns, and
    out[row, e * ff + c] = gates[row, e] * silu(gate) * up."""
    _dev(z, "z"), _dev(gates, "gates"), _dev(out, "out")
    rows, experts = gates.shape
    if form not in ("relu_squared", "silu_gated"):
        raise KernelError(f"routed_act: unknown form {form!r}")
    per = 2 if form == "silu_gated" else 1
    if (gates.dtype != torch.float32 or z.dim() != 2 or z.shape[0] != rows or z.shape[1] % max(per * experts, 1)
            or tuple(out.shape) != (rows, z.shape[1] // per) or not z.is_contiguous() or not out.is_contiguous()):
        raise KernelError(f"routed_act: z {tuple(z.shape)} and out {tuple(out.shape)} against gates {tuple(gates.shape)}")
    lib = sublayer()
    _check(lib, lib.nnis_routed_act(z.data_ptr(), _code(z), gates.data_ptr(), out.data_ptr(), _code(out), rows, experts,
                                    z.shape[1] // (per * experts), per - 1, _stream()))
    return out


def rows_axpy(y: torch.Tensor, h: torch.Tensor, keep: torch.Tensor) -> torch.Tensor:
    """y[row] += keep[row] * h[row]."""
    _dev(y, "y"), _dev(h, "h"), _dev(keep, "keep")
    if y.dim() != 2 or h.shape != y.shape or keep.dtype != torch.float32 or keep.numel() != y.shape[0]:
        raise KernelError(f"rows_axpy: y {tuple(y.shape)}, h {tuple(h.shape)}, a float32 factor per row")
    lib = sublayer()
    _check(lib, lib.nnis_rows_axpy(y.data_ptr(), _code(y), h.data_ptr(), _code(h), keep.data_ptr(), y.shape[0], y.shape[1], _stream()))
    return y


def sigmoid_gate(o: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """o *= sigmoid(gate) element by element; ``gate``: a view [rows, width] whose rows may be further apart."""
    _dev(o, "o")
    if not gate.is_cuda or gate.shape != o.shape or o.dim() != 2 or (gate.shape[1] > 1 and gate.stride(1) != 1):
        raise KernelError(f"sigmoid_gate: o {tuple(o.shape)} against a gate {tuple(gate.shape)} with adjacent columns")
    lib = sublayer()
    _check(lib, lib.nnis_sigmoid_gate(o.data_ptr(), _code(o), gate.data_ptr(), _code(gate), gate.stride(0) if o.shape[0] > 1 else o.shape[1],
                                      o.shape[0], o.shape[1], _stream()))
    return o


HEAD_NORM_MOST_CHANNELS = 1024


def head_norm_write(rows: torch.Tensor, columns, q_out: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                    eps: float, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rot_dim: int, neighbours: bool,
                    tok_slot: torch.Tensor, tok_pos: torch.Tensor, k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor],
                    block_table: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int, value_dim: int) -> torch.Tensor:
    """Queries and keys of a fused projection's ``rows`` head by head: an RMS norm over the head with a weight that the
    heads share (None: no norm), then the rotation of the first ``rot_dim`` channels by the token's position (channel
    2i with 2i + 1 if ``neighbours``, else i with i + rot_dim / 2); queries to ``q_out``, keys and values into the
    pages.  ``columns``: (first column of the queries, of the keys, of the values) in a row; with ``k_pages`` None the
    rows bring queries only."""
    _dev(rows, "rows"), _dev(q_out, "q_out"), _dev(tok_slot, "tok_slot"), _dev(tok_pos, "tok_pos")
    tokens = rows.shape[0]
    q_col, k_col, v_col = columns
    keys = kv_heads if k_pages is not None else 0
    need = max(q_col + heads * head_dim, (k_col + keys * head_dim) if keys else 0, (v_col + keys * value_dim) if keys else 0)
    if rows.dim() != 2 or rows.shape[1] < need or tuple(q_out.shape) != (tokens, heads * head_dim):
        raise KernelError(f"head_norm_write: rows {tuple(rows.shape)} / q_out {tuple(q_out.shape)} do not fit {heads}+{keys} heads of {head_dim}")
    if tok_slot.dtype != torch.int32 or tok_pos.dtype != torch.int32 or tok_slot.numel() < tokens or tok_pos.numel() < tokens:
        raise KernelError("head_norm_write: tok_slot / tok_pos must be int32 with one entry per token")
    if head_dim > HEAD_NORM_MOST_CHANNELS:
        raise KernelError(f"head_norm_write: heads of up to {HEAD_NORM_MOST_CHANNELS} channels, got {head_dim}")
    w_code = 0
    for weight in (q_weight, k_weight):
        if weight is not None:
            _dev(weight, "head norm weight")
            if weight.numel() != head_dim:
                raise KernelError(f"head_norm_write: a norm weight of {weight.numel()} for heads of {head_dim}")
            w_code = _code(weight)
    if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
        raise KernelError("head_norm_write: the two norm weights differ in type")
    table_positions = 0
    if cos is not None:
        _dev(cos, "cos"), _dev(sin, "sin")
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[1] != rot_dim // 2:
            raise KernelError(f"head_norm_write: tables {tuple(cos.shape)} do not fit rot_dim {rot_dim} in float32")
        table_positions = cos.shape[0]
    max_pages = cache_code = 0
    if keys:
        _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"), _dev(block_table, "block_table")
        if not _pages_fit(k_pages, v_pages, kv_heads, head_dim, value_dim):
            raise KernelError(f"head_norm_write: page shapes {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not fit")
        if block_table.dtype != torch.int32 or block_table.dim() != 2:
            raise KernelError("head_norm_write: block_table must be int32 [slots, pages]")
        max_pages, cache_code = block_table.shape[1], _code(k_pages)
    lib = sublayer()
    _check(lib, lib.nnis_head_norm_write(rows.data_ptr(), _code(rows), rows.stride(0) if tokens > 1 else rows.shape[1], q_col,
                                         k_col if keys else -1, v_col if keys else -1, q_out.data_ptr(), _code(q_out), _ptr(q_weight),
                                         _ptr(k_weight), w_code, float(eps), _ptr(cos), _ptr(sin), table_positions, int(rot_dim),
                                         1 if neighbours else 0, tok_slot.data_ptr(), tok_pos.data_ptr(), _ptr(k_pages) if keys else None,
                                         _ptr(v_pages) if keys else None, cache_code, _ptr(block_table) if keys else None, max_pages,
                                         tokens, heads, keys, head_dim, int(value_dim), _stream()))
    return q_out


def pool_blocks(k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor, pooled: PooledBlocks, ctx, kv_heads: int,
                head_dim: int, value_dim: int) -> None:
    """For every block of ``pooled.pool`` tokens that the step ``ctx`` completes in one of its sequences: the mean of
    the block's keys and the mean of its values, as the pages hold them, into the block's entry of ``pooled``."""
    for t, what in ((k_pages, "k_pages"), (v_pages, "v_pages"), (block_table, "block_table")):
        _dev(t, what)
    pooled.check(k_pages, v_pages, kv_heads, head_dim, value_dim, window=1)
    if not _pages_fit(k_pages, v_pages, kv_heads, head_dim, value_dim):
        raise KernelError(f"pool_blocks: page shapes {tuple(k_pages.shape)} / {tuple(v_pages.shape)} do not fit")
    _step_arrays(ctx, "pool_blocks")
    _dev(ctx.seq_pos0, "step metadata")
    if ctx.seq_pos0.dtype != torch.int32 or ctx.seq_pos0.numel() < ctx.batch:
        raise KernelError("pool_blocks: the step's first positions must be int32, one a sequence")
    lib = sublayer()
    _check(lib, lib.nnis_pool_blocks(k_pages.data_ptr(), v_pages.data_ptr(), _code(k_pages), block_table.data_ptr(), block_table.shape[1],
                                     pooled.k_pages.data_ptr(), pooled.v_pages.data_ptr(), pooled.block_table.data_ptr(),
                                     pooled.block_table.shape[1], ctx.seq_slot.data_ptr(), ctx.seq_start.data_ptr(),
                                     ctx.seq_pos0.data_ptr(), ctx.batch, ctx.tokens, kv_heads, head_dim, int(value_dim), pooled.pool, _stream()))


def min_gru(rows: torch.Tensor, z_bias: Optional[torch.Tensor], x_bias: Optional[torch.Tensor], state: torch.Tensor, ctx,
            out: torch.Tensor) -> torch.Tensor:
    """The minGRU recurrence over each sequence's tokens, from and into ``state`` (float32 [slots, width]): with ``rows``
    [tokens, 3 * width] = (zp | up | g): z = sigmoid(zp + z_bias), u = up + x_bias, c = u + 1/2 where u >= 0 and
    sigmoid(u) below, S <- (1 - z) S + z c, out = S * silu(g)."""
    _dev(rows, "rows"), _dev(state, "state"), _dev(out, "out")
    tokens, width = out.shape
    if rows.dim() != 2 or rows.shape[0] != tokens or rows.shape[1] < 3 * width:
        raise KernelError(f"min_gru: rows {tuple(rows.shape)} do not hold three times the {width} channels of out {tuple(out.shape)}")
    if state.dtype != torch.float32 or tuple(state.shape[1:]) != (width,):
        raise KernelError(f"min_gru: state must be float32 [slots, {width}], got {tuple(state.shape)} {state.dtype}")
    if (z_bias is None) != (x_bias is None):
        raise KernelError("min_gru: both biases or none")
    if z_bias is not None:
        _dev(z_bias, "z_bias"), _dev(x_bias, "x_bias")
        if z_bias.numel() != width or x_bias.numel() != width or z_bias.dtype != x_bias.dtype:
            raise KernelError("min_gru: the biases have one entry per channel and one type")
    _step_arrays(ctx, "min_gru")
    piece, pieces = run_pieces(ctx, width * 8)
    decay = ends = None
    if pieces > 1:
        scratch = torch.empty(2, ctx.batch * pieces * width, dtype=torch.float32, device=rows.device)
        decay, ends = scratch[0], scratch[1]
    lib = recurrent()
    _check(lib, lib.nnis_min_gru(rows.data_ptr(), _code(rows), rows.stride(0) if tokens > 1 else rows.shape[1], _ptr(z_bias), _ptr(x_bias),
                                 _code(z_bias) if z_bias is not None else 0, state.data_ptr(), ctx.seq_slot.data_ptr(),
                                 ctx.seq_start.data_ptr(), ctx.batch, width, out.data_ptr(), _code(out), piece, pieces, _ptr(decay),
                                 _ptr(ends), _stream()))
    return out
