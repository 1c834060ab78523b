"""Python faces of the HIP kernels: shape/dtype checks on the host, then one
C call on the current torch stream.  Nothing here computes on the CPU and there
is no alternative implementation behind these functions."""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from . import arena, library
from .arena import empty

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}

_c_i64 = ctypes.c_int64
_c_int = ctypes.c_int
_c_f = ctypes.c_float
_c_p = ctypes.c_void_p

_configured = False


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _CODE[dtype]
    except KeyError:
        raise TypeError(f"the kernels store float32 or bfloat16, not {dtype}") from None


def _lib():
    global _configured
    lib = library.load()
    if not _configured:
        lib.st_last_error.restype = ctypes.c_char_p
        lib.st_hash_uniform.restype = ctypes.c_float
        lib.st_hash_uniform.argtypes = [ctypes.c_uint32] * 4
        lib.st_lookup.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_p, _c_int, _c_int, _c_int,
                                  _c_int, _c_int, _c_int, _c_p]
        lib.st_layernorm.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_f, _c_int, _c_int, _c_p]
        lib.st_kv_write.argtypes = [_c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_int,
                                    _c_int, _c_int, _c_int, _c_int, _c_int, _c_p]
        lib.st_cast.argtypes = [_c_p, _c_p, _c_i64, _c_int, _c_int, _c_p]
        lib.st_activation_multiply.argtypes = [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_int, _c_int, _c_int,
                                               _c_int, _c_p]
        lib.st_gemm.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                _c_int, _c_int, _c_p, _c_p]
        lib.st_gemm_path_counts.argtypes = [_c_p, _c_int]
        lib.st_gemm_library_rule.argtypes = [_c_int, _c_i64, _c_int]
        lib.st_gemm_can_fuse_norm.argtypes = [_c_int, _c_int, _c_int, _c_int]
        lib.st_gemm_wide_offered.argtypes = [_c_int, _c_int, _c_int, _c_int]
        lib.st_gemm_can_fuse_merge.argtypes = [_c_int] * 7
        lib.st_gemm_library_tuning.argtypes = [_c_int]
        lib.st_attn_rows.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_p,
                                     _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_f, _c_int, _c_f, _c_int,
                                     _c_int, _c_int, _c_p]
        lib.st_attn_prefill.argtypes = [_c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_int,
                                        _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                        _c_f, _c_int, _c_f, _c_int, _c_int, _c_int, _c_int, _c_p]
        lib.st_attn_prefill_tile_rows.argtypes = [_c_int] * 6
        lib.st_probe_read.argtypes = [_c_p, _c_i64, _c_p, _c_int, _c_int, _c_p]
        lib.st_probe_empty.argtypes = [_c_p, _c_p]
        lib.st_probe_fill.argtypes = [_c_p, _c_i64, _c_p, _c_int, _c_int, _c_int, _c_p]
        lib.st_probe_mfma.argtypes = [_c_p, _c_int, _c_int, _c_int, _c_p]
        lib.st_sample.argtypes = [_c_p, _c_p, _c_int, _c_int, _c_p, _c_p, _c_p, _c_p]
        lib.st_token_conv.argtypes = [_c_p, _c_p, _c_i64, _c_int, _c_p, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_int,
                                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_p]
        lib.st_token_conv_state.argtypes = [_c_p, _c_i64, _c_p, _c_i64, _c_int, _c_p, _c_p, _c_p, _c_int, _c_int,
                                            _c_int, _c_p]
        lib.st_rotary.argtypes = [_c_p, _c_i64, _c_int, _c_p, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_p, _c_f,
                                  _c_p, _c_int, _c_int, _c_p]
        lib.st_paged_write.argtypes = [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int,
                                       _c_int, _c_int, _c_f, _c_int, _c_p]
        lib.st_concat_cast.argtypes = [_c_p, _c_p, _c_int, _c_p, _c_int, _c_int, _c_int, _c_p]
        lib.st_sink_attention_lds.restype = _c_i64
        lib.st_sink_attention_lds.argtypes = [_c_int, _c_int, _c_int]
        lib.st_sink_attention.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p,
                                          _c_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_f, _c_int,
                                          _c_int, _c_int, _c_int, _c_int, _c_p]
        lib.st_recurrence_gates.argtypes = [_c_p, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_int, _c_int, _c_int, _c_p]
        lib.st_unit_norm.argtypes = [_c_p, _c_i64, _c_int, _c_int, _c_int, _c_f, _c_f, _c_p]
        lib.st_state_scan.argtypes = [_c_p, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64,
                                      _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_p]
        lib.st_gated_group_norm.argtypes = [_c_p, _c_p, _c_p, _c_i64, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                            _c_int, _c_f, _c_int, _c_p]
        lib.st_decay_gate.argtypes = [_c_p, _c_p, _c_i64, _c_f, _c_p]
        lib.st_gla_scan.argtypes = [_c_p, _c_i64, _c_int, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p,
                                    _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_f, _c_int, _c_p]
        lib.st_gated_head_norm.argtypes = [_c_p, _c_p, _c_int, _c_i64, _c_p, _c_i64, _c_p, _c_int, _c_int, _c_int,
                                           _c_f, _c_int, _c_p]
        lib.st_latent_write.argtypes = [_c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int,
                                        _c_int, _c_int, _c_f, _c_int, _c_p, _c_f, _c_int, _c_p]
        lib.st_moe_route.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_p]
        lib.st_moe_align.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_p]
        lib.st_moe_up.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                  _c_f, _c_int, _c_int, _c_p]
        lib.st_moe_down.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int,
                                    _c_f, _c_int, _c_p]
        lib.st_moe_combine.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_f, _c_p]
        lib.st_dynamic_tanh.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int,
                                        _c_int, _c_p]
        lib.st_unit_add.argtypes = [_c_p, _c_p, _c_p, _c_int, _c_int, _c_f, _c_p]
        lib.st_retention_chunk_rows.argtypes = [_c_int]
        lib.st_retention_chunks.argtypes = [_c_p, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_f, _c_p, _c_i64,
                                            _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_p, _c_i64, _c_p]
        lib.st_token_side.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_i64, _c_int, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int,
                                      _c_f, _c_int, _c_p]
        lib.st_row_add.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_p]
        lib.st_scale_softcap.argtypes = [_c_p, _c_i64, _c_f, _c_f, _c_p]
        lib.st_streams_expand.argtypes = [_c_p, _c_p, _c_int, _c_int, _c_int, _c_p]
        lib.st_streams_sum.argtypes = [_c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_p]
        lib.st_streams_read.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_f, _c_int, _c_p]
        lib.st_streams_write.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int, _c_f, _c_int,
                                         _c_p]
        lib.st_hashed_embed.argtypes = [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int, _c_int, _c_int,
                                        _c_int, _c_i64, _c_i64, _c_f, _c_int, _c_int, _c_p]
        lib.st_qk_norm_write.argtypes = [_c_p, _c_p, _c_p, _c_i64, _c_p, _c_i64, _c_p, _c_p, _c_p, _c_p, _c_p, _c_int,
                                         _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_f, _c_int, _c_int, _c_p]
        if torch.cuda.is_available():
            lib.st_gemm_library_init()  # handle and workspace exist before any stream capture
        _configured = True
    return lib


class KernelError(RuntimeError):
    pass


# A KernelTimer (ops/profile.py) while one is active, else None.  Every face below reports its
# call to it: the timer brackets the call with two events on the current stream.
_timer = None


def _timed(name: str, describe):
    """Decorator of a kernel face: with a timer active, the call is bracketed by events and
    recorded under ``name`` with ``describe(*args, **kwargs)`` (a dict of sizes)."""
    def wrap(fn):
        def face(*args, **kwargs):
            if _timer is None:
                return fn(*args, **kwargs)
            begin = _timer.begin()
            out = fn(*args, **kwargs)
            _timer.end(name, describe(*args, **kwargs), begin)
            return out
        face.__name__, face.__doc__ = fn.__name__, fn.__doc__
        return face
    return wrap


# ST_AMD_DEBUG_SYNC=1: wait for the device after every kernel call and surface its errors there
# (the reference's DEBUG build does the same after every launch, src/csrc/util/cuda_utils.h:19-31)
_DEBUG_SYNC = os.environ.get("ST_AMD_DEBUG_SYNC", "") not in ("", "0")


def _check(rc: int) -> None:
    if rc != 0:
        raise KernelError(_lib().st_last_error().decode("utf-8", "replace"))
    if _DEBUG_SYNC and not torch.cuda.is_current_stream_capturing():
        torch.cuda.synchronize()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_index: Optional[int] = None


def _stream() -> int:
    """The current HIP stream's handle.  Asked for at every kernel call (a caller may have
    switched streams, e.g. to record a step), so by the cheapest route torch offers."""
    global _device_index
    if _raw_stream is None:
        return torch.cuda.current_stream().cuda_stream
    if _device_index is None:
        _device_index = torch.cuda.current_device()     # one GPU per process
    return _raw_stream(_device_index)


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(t: torch.Tensor, name: str, dtype=None, shape=None, contiguous=True) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name} must be a GPU tensor")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    if contiguous and not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")


# ------------------------------------------------------------------------ lookup
def _d_lookup(ids, table, *, add_ids=None, add_table=None, out_f32=None, out_t=None, **kw):
    ref = table if table is not None else add_table
    idx = ids if ids is not None else add_ids
    n, width = idx.shape[0], ref.shape[1]
    tables = (table is not None) + (add_table is not None)
    return {"rows": n, "width": width,
            "bytes": n * width * (tables * ref.element_size() + 4 * (out_f32 is not None) +
                                  ref.element_size() * (out_t is not None))}


@_timed("lookup", _d_lookup)
def lookup(ids: Optional[torch.Tensor], table: Optional[torch.Tensor], *,
           add_ids: Optional[torch.Tensor] = None, add_offset: int = 0,
           add_table: Optional[torch.Tensor] = None, out_f32: Optional[torch.Tensor] = None,
           out_t: Optional[torch.Tensor] = None, accumulate: bool = False) -> None:
    """out[t] = (out[t] if accumulate) + table[ids[t]] + add_table[add_ids[t] + add_offset];
    an index outside its table adds nothing."""
    ref = table if table is not None else add_table
    if ref is None:
        raise KernelError("lookup needs a table")
    width = ref.shape[1]
    idx = ids if ids is not None else add_ids
    n = idx.shape[0]
    if table is not None:
        _need(table, "table", shape=(table.shape[0], width))
        _need(ids, "ids", torch.int32, (n,))
    if add_table is not None:
        _need(add_table, "add_table", ref.dtype, (add_table.shape[0], width))
        _need(add_ids, "add_ids", torch.int32, (n,))
    if out_f32 is not None:
        _need(out_f32, "out_f32", torch.float32, (n, width))
    if out_t is not None:
        _need(out_t, "out_t", ref.dtype, (n, width))
    _check(_lib().st_lookup(_ptr(out_f32), _ptr(out_t), _ptr(ids), _ptr(table), _ptr(add_ids),
                            int(add_offset), _ptr(add_table),
                            table.shape[0] if table is not None else 0,
                            add_table.shape[0] if add_table is not None else 0, n, width, int(accumulate),
                            dtype_code(ref.dtype), _stream()))


# --------------------------------------------------------------------- LayerNorm
def _d_layernorm(x, gamma, beta, eps, *, rows=None, out_t=None, out_f32=None, center=True):
    n = rows.shape[0] if rows is not None else x.shape[0]
    w = x.shape[-1]
    return {"rows": n, "width": w,
            "bytes": n * w * (4 + (out_t.element_size() if out_t is not None else 0) + 4 * (out_f32 is not None))}


@_timed("layernorm", _d_layernorm)
def layernorm(x: torch.Tensor, gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor],
              eps: float, *, rows: Optional[torch.Tensor] = None,
              out_t: Optional[torch.Tensor] = None, out_f32: Optional[torch.Tensor] = None,
              center: bool = True) -> None:
    """LayerNorm over the last dimension of float rows; row r reads x[rows[r]] if given.
    ``center=False``: no mean is taken off (root-mean-square norm)."""
    _need(x, "x", torch.float32)
    width = x.shape[-1]
    n = rows.shape[0] if rows is not None else x.shape[0]
    if rows is not None:
        _need(rows, "rows", torch.int32, (n,))
    for name, v in (("gamma", gamma), ("beta", beta)):
        if v is not None:
            _need(v, name, torch.float32, (width,))
    if out_t is None and out_f32 is None:
        raise KernelError("layernorm needs a destination")
    code = F32
    if out_t is not None:
        _need(out_t, "out_t", None, (n, width))
        code = dtype_code(out_t.dtype)
    if out_f32 is not None:
        _need(out_f32, "out_f32", torch.float32, (n, width))
        if rows is not None and out_f32.data_ptr() == x.data_ptr():
            raise KernelError("layernorm: a gathered LayerNorm cannot write over its input")
    _check(_lib().st_layernorm(_ptr(out_t), _ptr(out_f32), _ptr(x), _ptr(rows), _ptr(gamma), _ptr(beta),
                               n, width, float(eps), int(bool(center)), code, _stream()))


# -------------------------------------------------------------------------- GEMM
class _GemmExtras(ctypes.Structure):
    """Mirror of StGemmExtras (csrc/gemm_extras.h)."""
    _fields_ = [("ln_x", _c_p), ("ln_gamma", _c_p), ("ln_beta", _c_p), ("ln_eps", _c_f), ("ln_no_center", _c_int),
                ("k_cache", _c_p), ("v_cache", _c_p), ("page_stride", _c_i64), ("token_item", _c_p),
                ("positions", _c_p), ("block_table", _c_p), ("max_pages", _c_int), ("page_size", _c_int),
                ("q_size", _c_int), ("kv_size", _c_int), ("head_dim", _c_int), ("_pad1", _c_int),
                ("mg_o", _c_p), ("mg_lse", _c_p), ("mg_splits", _c_int), ("mg_heads", _c_int),
                ("mg_head_dim", _c_int), ("_pad2", _c_int),
                ("ln_rows", _c_p), ("best_ids", _c_p), ("best_val", _c_p), ("best_idx", _c_p),
                ("out_scale", _c_f), ("_pad3", _c_int)]


class KvScatter:
    """Where a fused QKV product also stores the new keys and values: the layer's cache views,
    the step's row -> (item, position) arrays and the block table."""

    def __init__(self, k_cache: torch.Tensor, v_cache: torch.Tensor, token_item: torch.Tensor,
                 positions: torch.Tensor, block_table: torch.Tensor, q_size: int):
        self.k_cache, self.v_cache = k_cache, v_cache
        self.token_item, self.positions, self.block_table = token_item, positions, block_table
        self.q_size = q_size


class NormInput:
    """The input of a product given as (float rows, gain, bias, eps): the product normalises
    the rows itself.  With ``rows`` (int32 [M] on the device) row m of the input is the norm of
    ``x32[rows[m]]`` (where ``wide_offered``).  ``center=False``: the root-mean-square norm (no
    mean is taken off)."""

    def __init__(self, x32: torch.Tensor, gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor],
                 eps: float, rows: Optional[torch.Tensor] = None, center: bool = True):
        self.x32, self.gamma, self.beta, self.eps, self.rows, self.center = x32, gamma, beta, eps, rows, center


class SplitAttention:
    """The input of a product given as an attention output still split over the keys:
    ``part_o`` [M, heads, splits, head_dim] normalised partial results and ``part_lse``
    [M, heads, splits] their log-sum-exps (``attention_rows(..., merge=False)``).  The product
    merges the splits itself."""

    def __init__(self, part_o: torch.Tensor, part_lse: torch.Tensor):
        self.part_o, self.part_lse = part_o, part_lse


def can_fuse_merge(M: int, N: int, K: int, splits: int, heads: int, head_dim: int, dtype: torch.dtype) -> bool:
    """Whether ``gemm`` takes a ``SplitAttention`` for this shape."""
    return bool(_lib().st_gemm_can_fuse_merge(M, N, K, splits, heads, head_dim, dtype_code(dtype)))


class tuned_products:
    """``with tuned_products():`` the vendor library's candidate kernels are timed for every
    product shape issued inside (outside stream capture) and the fastest kept for that shape from
    then on.  For the preparation of steps that are replayed many times; ~20 ms a shape."""

    def __enter__(self):
        _lib().st_gemm_library_tuning(1)
        return self

    def __exit__(self, *exc):
        torch.cuda.synchronize()
        _lib().st_gemm_library_tuning(0)
        return False


GEMM_PATHS = ("library", "generic_f32", "generic_bf16", "resident", "resident_norm", "resident_merge",
              "resident_staged", "skinny16", "skinny32", "skinny64", "tiled_mfma", "wide")


def gemm_path_counts(reset: bool = False) -> dict:
    """Calls of ``gemm`` per kernel family since the last reset: which dispatch branches ran."""
    n = len(GEMM_PATHS)
    buf = (ctypes.c_uint64 * n)()
    got = _lib().st_gemm_path_counts(buf, int(reset))
    if got != n:
        raise KernelError(f"the library counts {got} product paths, this module names {n}")
    return {name: int(buf[i]) for i, name in enumerate(GEMM_PATHS)}


def gemm_library_rule(min_rows: int = -1, min_weights: int = -1, min_depth: int = -1) -> None:
    """Change when bfloat16 products go to the vendor library (for measurements): from ``min_rows``
    rows on, and below that for matrices of ``min_weights`` elements and ``min_depth`` depth.  -1
    leaves a setting, -2 puts its fitted default back (``gemm_library_rule(-2, -2, -2)``: all of
    them).  A step recorded before the change keeps its kernels."""
    _lib().st_gemm_library_rule(int(min_rows), int(min_weights), int(min_depth))


def gemm_wide_workgroups(mode: int = 3) -> None:
    """Which workgroup shapes a product with the norm prologue may take (for measurements and
    tests): 0 only 16 features a workgroup, 1 also 24 with 8 waves, 3 (the default) 24 or 32 with 16 waves,
    7 the same with 32 tried first; a negative number puts the default back."""
    _lib().st_gemm_wide_workgroups(int(mode))


def can_fuse_norm(M: int, N: int, K: int, dtype: torch.dtype) -> bool:
    """Whether ``gemm`` takes a ``NormInput`` (without a row index) for this shape."""
    return bool(_lib().st_gemm_can_fuse_norm(M, N, K, dtype_code(dtype)))


def wide_offered(M: int, N: int, K: int, dtype: torch.dtype) -> bool:
    """Whether ``gemm(..., out_f32=True)`` runs this plain product in the persistent kernel for few
    rows and a very wide matrix (an output head): the kernel that takes a ``NormInput`` with a row
    index and fills ``best``."""
    return bool(_lib().st_gemm_wide_offered(M, N, K, dtype_code(dtype)))


# functions of the products' epilogues and of ``activation_multiply``, by the C interface's number
# (csrc/activation.h; the names config files use for them)
ACTIVATIONS = {"none": 0, "relu": 1, "silu": 2, "gelu_tanh": 3, "gelu_new": 3, "gelu": 4, "gelu_erf": 4,
               "relu_squared": 5, "relu2": 5, "sigmoid": 6}


def _d_gemm(x, w, *, bias=None, residual=None, activation="none", out=None, out_f32=False, algo=0,
            kv_scatter=None, best=None, out_scale=1.0):
    N, K = w.shape
    fused = []
    if isinstance(x, NormInput):
        M = x.rows.shape[0] if x.rows is not None else x.x32.shape[0]
        in_bytes = M * K * 4
        fused.append("norm")
    elif isinstance(x, SplitAttention):
        M, in_bytes = x.part_o.shape[0], x.part_o.numel() * 4
        fused.append("merge")
    else:
        M, in_bytes = x.shape[0], x.shape[0] * K * w.element_size()
    if kv_scatter is not None:
        fused.append("kv")
    if best is not None:
        fused.append("best")
    if activation != "none":
        fused.append(activation)
    if residual is not None:
        fused.append("residual")
    out_elem = 4 if (out_f32 or w.dtype == torch.float32) else w.element_size()
    return {"M": M, "N": N, "K": K, "fused": "+".join(fused), "dtype": str(w.dtype).replace("torch.", ""),
            "bytes": N * K * w.element_size() + in_bytes + M * N * (out_elem + 4 * (residual is not None)),
            "flops": 2 * M * N * K}


@_timed("gemm", _d_gemm)
def gemm(x, w: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
         residual: Optional[torch.Tensor] = None, activation: str = "none",
         out: Optional[torch.Tensor] = None, out_f32: bool = False, algo: int = 0,
         kv_scatter: Optional[KvScatter] = None, best: Optional[torch.Tensor] = None,
         out_scale: float = 1.0) -> torch.Tensor:
    """out[M,N] = out_scale * act(x[M,K] @ w[N,K]^T (+bias)) (+residual); float accumulation.
    ``activation`` is one of ``ACTIVATIONS``.

    ``x`` is a tensor of w's dtype, a ``NormInput`` (where ``can_fuse_norm``) or a
    ``SplitAttention`` (where ``can_fuse_merge``).  With
    ``kv_scatter`` the output features after the first q_size are also written into the
    cache pages (w then is a fused q|k|v matrix).  ``best`` (int32 [M], where ``wide_offered``):
    receives the index of every row's largest output, the lowest on ties."""
    N, K = w.shape
    _need(w, "w", None, (N, K))
    code = dtype_code(w.dtype)
    if activation not in ACTIVATIONS:
        raise KernelError(f"the products' epilogues know {sorted(ACTIVATIONS)}, not {activation!r}")
    ex = None
    keep = []
    if isinstance(x, NormInput):
        M = x.x32.shape[0]
        _need(x.x32, "norm input", torch.float32, (M, K))
        for name, v in (("gamma", x.gamma), ("beta", x.beta)):
            if v is not None:
                _need(v, name, torch.float32, (K,))
        ex = _GemmExtras()
        ex.ln_x, ex.ln_gamma, ex.ln_beta, ex.ln_eps = _ptr(x.x32), _ptr(x.gamma), _ptr(x.beta), float(x.eps)
        ex.ln_no_center = 0 if x.center else 1
        if x.rows is not None:
            M = x.rows.shape[0]
            _need(x.rows, "row index", torch.int32, (M,))
            ex.ln_rows = _ptr(x.rows)
        x_ptr, device = None, x.x32.device
    elif isinstance(x, SplitAttention):
        M, heads, splits, hd = x.part_o.shape
        _need(x.part_o, "partial outputs", torch.float32, (M, heads, splits, hd))
        _need(x.part_lse, "log-sum-exps", torch.float32, (M, heads, splits))
        if heads * hd != K:
            raise KernelError(f"{heads} heads of {hd} do not make the product's {K} inputs")
        ex = _GemmExtras()
        ex.mg_o, ex.mg_lse = _ptr(x.part_o), _ptr(x.part_lse)
        ex.mg_splits, ex.mg_heads, ex.mg_head_dim = splits, heads, hd
        x_ptr, device = None, x.part_o.device
    else:
        M = x.shape[0]
        _need(x, "x", w.dtype, (M, K))
        x_ptr, device = x.data_ptr(), x.device
    odt = torch.float32 if (out_f32 or code == F32) else w.dtype
    if out is None:
        out = empty((M, N), odt, device)
    _need(out, "out", odt, (M, N))
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,))
    if residual is not None:
        _need(residual, "residual", torch.float32, (M, N))
    if kv_scatter is not None:
        ks = kv_scatter
        num_pages, nkv, ps, hd = _check_cache(ks.k_cache, ks.v_cache, out)
        _need(ks.token_item, "token_item", torch.int32, (M,))
        _need(ks.positions, "positions", torch.int32, (M,))
        _need(ks.block_table, "block_table", torch.int32)
        if ex is None:
            ex = _GemmExtras()
        ex.k_cache, ex.v_cache, ex.page_stride = _ptr(ks.k_cache), _ptr(ks.v_cache), ks.k_cache.stride(0)
        ex.token_item, ex.positions, ex.block_table = _ptr(ks.token_item), _ptr(ks.positions), _ptr(ks.block_table)
        ex.max_pages, ex.page_size = ks.block_table.shape[1], ps
        ex.q_size, ex.kv_size, ex.head_dim = ks.q_size, nkv * hd, hd
    if best is not None:
        _need(best, "best", torch.int32, (M,))
        n_scratch = 16 * _lib().st_gemm_wide_groups()
        if ex is None:
            ex = _GemmExtras()
        val = empty((n_scratch,), torch.float32, device)
        idx = empty((n_scratch,), torch.int32, device)
        keep += [val, idx]
        ex.best_ids, ex.best_val, ex.best_idx = _ptr(best), _ptr(val), _ptr(idx)
    if float(out_scale) != 1.0:
        if ex is None:
            ex = _GemmExtras()
        ex.out_scale = float(out_scale)
    _check(_lib().st_gemm(_ptr(out), x_ptr, _ptr(w), _ptr(bias), _ptr(residual), M, N, K, ACTIVATIONS[activation],
                          code, int(odt == torch.float32), int(algo),
                          ctypes.byref(ex) if ex is not None else None, _stream()))
    return out


# ---------------------------------------------------------------------- KV write
def _d_kv_write(k_cache, v_cache, k_src, v_src, *a, **kw):
    return {"rows": k_src.shape[0], "width": k_src.shape[1], "bytes": 4 * k_src.numel() * k_src.element_size()}


@_timed("kv_write", _d_kv_write)
def kv_write(k_cache: torch.Tensor, v_cache: torch.Tensor, k_src: torch.Tensor, v_src: torch.Tensor,
             token_item: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
             page_size: int) -> None:
    """Copy each token's key/value heads into its page.

    k_cache/v_cache: [num_pages, num_kv_heads, page_size, head_dim] views (the page
    dimension may be strided).  k_src/v_src: [T, num_kv_heads*head_dim] views with a
    common row stride (e.g. column slices of the fused QKV output)."""
    num_pages, nkv, ps, hd = k_cache.shape
    if ps != page_size:
        raise KernelError(f"cache pages hold {ps} tokens, the step says {page_size}")
    T = k_src.shape[0]
    for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
        _need(c, name, k_cache.dtype, (num_pages, nkv, ps, hd), contiguous=False)
        if c.stride()[1:] != (ps * hd, hd, 1):
            raise KernelError(f"{name}: a page must be contiguous")
    if k_cache.stride(0) != v_cache.stride(0):
        raise KernelError("k_cache and v_cache must share the page stride")
    for name, s in (("k_src", k_src), ("v_src", v_src)):
        _need(s, name, k_cache.dtype, (T, nkv * hd), contiguous=False)
        if s.stride(1) != 1 or s.stride(0) != k_src.stride(0):
            raise KernelError(f"{name}: rows must be dense with a common stride")
    _need(token_item, "token_item", torch.int32, (T,))
    _need(positions, "positions", torch.int32, (T,))
    _need(block_table, "block_table", torch.int32)
    _check(_lib().st_kv_write(_ptr(k_cache), _ptr(v_cache), k_cache.stride(0), _ptr(k_src), _ptr(v_src),
                              k_src.stride(0), _ptr(token_item), _ptr(positions), _ptr(block_table),
                              block_table.shape[1], ps, T, nkv, hd, dtype_code(k_cache.dtype), _stream()))


# --------------------------------------------------------------------- attention
def _check_cache(k_cache, v_cache, q):
    num_pages, nkv, ps, hd = k_cache.shape
    for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
        _need(c, name, q.dtype, (num_pages, nkv, ps, hd), contiguous=False)
        if c.stride()[1:] != (ps * hd, hd, 1):
            raise KernelError(f"{name}: a page must be contiguous")
    if k_cache.stride(0) != v_cache.stride(0):
        raise KernelError("k_cache and v_cache must share the page stride")
    return num_pages, nkv, ps, hd


def _d_attention_rows(q, k_cache, v_cache, token_item, positions, block_table, num_q_heads, scale, *,
                      num_splits=1, row_ids=None, merge=True, **kw):
    # how many keys the rows read is on the device only: the caller of the timer knows its workload
    rows = row_ids.shape[0] if row_ids is not None else q.shape[0]
    info = {"rows": rows, "heads": num_q_heads, "kv_heads": k_cache.shape[1], "head_dim": k_cache.shape[3],
            "splits": num_splits, "merged": bool(merge), "elem": k_cache.element_size()}
    if kw.get("window"):
        info["window"] = int(kw["window"])       # negative: chunks of that many positions
    return info


def _d_attention_prefill(q, k_cache, v_cache, tile_item, *a, **kw):
    info = {"rows": q.shape[0], "tiles": tile_item.shape[0], "heads": q.shape[1] // k_cache.shape[3],
            "kv_heads": k_cache.shape[1], "head_dim": k_cache.shape[3], "elem": k_cache.element_size()}
    if kw.get("window"):
        info["window"] = int(kw["window"])
    return info


@_timed("attention_rows", _d_attention_rows)
def attention_rows(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   token_item: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
                   num_q_heads: int, scale: float, *, window: int = 0, num_splits: int = 1,
                   num_waves: int = 4, row_ids: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                   workspace: Optional[torch.Tensor] = None, merge: bool = True,
                   head_slopes: Optional[torch.Tensor] = None, softcap: float = 0.0):
    """Each query row attends over its request's cached keys [lo, position].

    q: [T, num_q_heads*head_dim] view (row stride free).  Returns [T, num_q_heads*head_dim];
    with ``row_ids`` only those batch rows are computed (and written).  ``merge=False`` (with
    num_splits > 1, all rows): the splits are left unmerged and returned as a
    ``SplitAttention`` for a product to merge.  ``head_slopes`` (float32 [num_q_heads]): a head's
    scaled scores get slope * (key position - query position) added.  ``window`` > 0: a row reads the last
    ``window`` positions; < 0: the positions of its own chunk of ``-window`` positions, chunks counted from
    the sequence's start.  ``softcap`` > 0: scaled scores pass through softcap * tanh(score / softcap)."""
    num_pages, nkv, ps, hd = _check_cache(k_cache, v_cache, q)
    T = q.shape[0]
    if head_slopes is not None:
        _need(head_slopes, "head_slopes", torch.float32, (num_q_heads,))
    _need(q, "q", None, (T, num_q_heads * hd), contiguous=False)
    if q.stride(1) != 1:
        raise KernelError("q rows must be dense")
    _need(token_item, "token_item", torch.int32, (T,))
    _need(positions, "positions", torch.int32, (T,))
    _need(block_table, "block_table", torch.int32)
    if not merge and (num_splits < 2 or row_ids is not None or T > 65535 or out is not None):
        raise KernelError("unmerged attention output needs splits, all rows and no destination")
    if merge:
        if out is None:
            out = empty((T, num_q_heads * hd), q.dtype, q.device)
        _need(out, "out", q.dtype, (T, num_q_heads * hd))
    n_rows = T
    if row_ids is not None:
        n_rows = row_ids.shape[0]
        _need(row_ids, "row_ids", torch.int32, (n_rows,))
    part_o = part_lse = None
    if num_splits > 1:
        n_o = min(n_rows, 65535) * num_q_heads * num_splits * hd
        n_l = min(n_rows, 65535) * num_q_heads * num_splits
        if workspace is None:
            workspace = empty((n_o + n_l,), torch.float32, q.device)
        _need(workspace, "workspace", torch.float32)
        if workspace.numel() < n_o + n_l:
            raise KernelError("attention workspace is too small")
        part_o, part_lse = workspace[:n_o], workspace[n_o:n_o + n_l]
    step = 65535
    for r0 in range(0, n_rows, step):
        r1 = min(n_rows, r0 + step)
        if row_ids is not None:
            o_ptr, q_ptr, ti_ptr, po_ptr = out.data_ptr(), q.data_ptr(), token_item.data_ptr(), positions.data_ptr()
            rid_ptr = row_ids[r0:r1].data_ptr()
        else:
            o_ptr, q_ptr = (out[r0:r1].data_ptr() if merge else None), q[r0:r1].data_ptr()
            ti_ptr, po_ptr = token_item[r0:r1].data_ptr(), positions[r0:r1].data_ptr()
            rid_ptr = None
        _check(_lib().st_attn_rows(
            o_ptr, _ptr(part_o), _ptr(part_lse), q_ptr, q.stride(0),
            _ptr(k_cache), _ptr(v_cache), k_cache.stride(0), rid_ptr, ti_ptr, po_ptr,
            _ptr(block_table), _ptr(head_slopes), block_table.shape[1], ps, r1 - r0,
            num_q_heads, nkv, hd, float(scale), int(window), float(softcap), int(num_splits), int(num_waves),
            dtype_code(q.dtype), _stream()))
    if not merge:
        return SplitAttention(part_o.view(T, num_q_heads, num_splits, hd), part_lse.view(T, num_q_heads, num_splits))
    return out


@_timed("attention_prefill", _d_attention_prefill)
def attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      tile_item: torch.Tensor, tile_q0: torch.Tensor,
                      item_tok_off: torch.Tensor, item_start: torch.Tensor, item_len: torch.Tensor,
                      block_table: torch.Tensor, num_q_heads: int, scale: float, *,
                      window: int = 0, out: Optional[torch.Tensor] = None, key_split: int = 0,
                      tile_rows: int = 64, algo: int = 0,
                      head_slopes: Optional[torch.Tensor] = None, softcap: float = 0.0) -> torch.Tensor:
    """Tiles of consecutive query rows of prompt portions attend over the cache.

    Tile i covers rows [tile_q0[i], tile_q0[i]+tile_rows) of item tile_item[i]; row r of an
    item sits at batch row item_tok_off[item]+r and at position item_start[item]+r.
    ``key_split``: groups of waves that share a tile's key blocks (1, 2 or 4; 0: chosen from
    the number of tiles).  ``tile_rows``: 64, or 128 where ``prefill_tile_rows`` says so.
    ``algo``: 0 chosen by the library, 1 the kernel that stages key blocks through registers,
    2 the kernel that loads them straight into LDS (it takes no ``head_slopes``, no ``softcap`` and no
    negative ``window``, which are as in ``attention_rows``)."""
    num_pages, nkv, ps, hd = _check_cache(k_cache, v_cache, q)
    T = q.shape[0]
    _need(q, "q", None, (T, num_q_heads * hd), contiguous=False)
    if q.stride(1) != 1:
        raise KernelError("q rows must be dense")
    nt = tile_item.shape[0]
    _need(tile_item, "tile_item", torch.int32, (nt,))
    _need(tile_q0, "tile_q0", torch.int32, (nt,))
    for name, v in (("item_tok_off", item_tok_off), ("item_start", item_start), ("item_len", item_len)):
        _need(v, name, torch.int32)
    _need(block_table, "block_table", torch.int32)
    if out is None:
        out = empty((T, num_q_heads * hd), q.dtype, q.device)
    _need(out, "out", q.dtype, (T, num_q_heads * hd))
    if head_slopes is not None:
        _need(head_slopes, "head_slopes", torch.float32, (num_q_heads,))
    _check(_lib().st_attn_prefill(
        _ptr(out), _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), k_cache.stride(0),
        _ptr(tile_item), _ptr(tile_q0), nt, _ptr(item_tok_off), _ptr(item_start), _ptr(item_len),
        _ptr(block_table), _ptr(head_slopes), block_table.shape[1], ps, num_q_heads, nkv, hd, float(scale), int(window),
        float(softcap), int(key_split), int(tile_rows), int(algo), dtype_code(q.dtype), _stream()))
    return out


PREFILL_TILE = 64   # query rows per tile of attention_prefill unless prefill_tile_rows says 128


def prefill_tile_rows(head_dim: int, page_size: int, max_pages: int, num_q_heads: int, num_rows: int,
                      dtype: torch.dtype) -> int:
    """Rows per tile (64 or 128) that ``attention_prefill`` serves best when ``num_rows`` query rows
    sit in items long enough for tiles."""
    return int(_lib().st_attn_prefill_tile_rows(head_dim, page_size, max_pages, num_q_heads, num_rows,
                                                dtype_code(dtype)))


def prefill_available() -> bool:
    """Whether the library holds the tiled (matrix-core) prompt attention kernel."""
    return bool(_lib().st_has_attn_prefill())


# ---------------------------------------------------------------------- sampling
def _d_sample(logits, **kw):
    return {"rows": logits.shape[0], "width": logits.shape[1], "bytes": logits.numel() * 4}


@_timed("sample", _d_sample)
def sample(logits: torch.Tensor, *, temperature: Optional[torch.Tensor] = None,
           seeds: Optional[torch.Tensor] = None, draws: Optional[torch.Tensor] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Token ids [R] (int32) from float logits [R,V]; rows with temperature <= 0 (or no
    temperature tensor) take the argmax, lowest index on ties."""
    R, V = logits.shape
    _need(logits, "logits", torch.float32, (R, V))
    if temperature is not None:
        _need(temperature, "temperature", torch.float32, (R,))
        _need(seeds, "seeds", torch.int32, (R, 2))
        _need(draws, "draws", torch.int32, (R,))
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _need(out, "out", torch.int32, (R,))
    _check(_lib().st_sample(_ptr(out), _ptr(logits), R, V, _ptr(temperature), _ptr(seeds), _ptr(draws),
                            _stream()))
    return out


def _d_cast(x, dtype, out=None):
    return {"rows": x.shape[0] if x.dim() else 1, "width": x.numel() // max(1, x.shape[0] if x.dim() else 1),
            "bytes": x.numel() * (x.element_size() + torch.empty((), dtype=dtype).element_size())}


@_timed("cast", _d_cast)
def cast(x: torch.Tensor, dtype: torch.dtype, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _need(x, "x")
    if out is None:
        out = empty(tuple(x.shape), dtype, x.device)
    _need(out, "out", dtype, x.shape)
    _check(_lib().st_cast(_ptr(out), _ptr(x), x.numel(), dtype_code(x.dtype), dtype_code(dtype), _stream()))
    return out


def _d_activation_multiply(a, b=None, activation="none", out=None):
    return {"rows": a.shape[0], "width": a.shape[1], "fused": activation,
            "bytes": a.numel() * a.element_size() * (2 + (b is not None))}


@_timed("activation_multiply", _d_activation_multiply)
def activation_multiply(a: torch.Tensor, b: Optional[torch.Tensor] = None, activation: str = "none",
                        out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = act(a) * b elementwise over [rows, width] (``b`` None: out = act(a)), float arithmetic.
    ``a``, ``b`` and ``out`` may be column slices of wider tensors (dense rows, any row stride), e.g.
    the two halves of one product's output; ``out`` may be ``a``."""
    if activation not in ACTIVATIONS:
        raise KernelError(f"the kernels know the activations {sorted(ACTIVATIONS)}, not {activation!r}")
    if a.dim() != 2:
        raise KernelError("activation_multiply takes [rows, width] tensors")
    rows, width = a.shape
    code = dtype_code(a.dtype)
    if out is None:
        out = empty((rows, width), a.dtype, a.device)
    for name, t in (("a", a), ("b", b), ("out", out)):
        if t is None:
            continue
        _need(t, name, a.dtype, (rows, width), contiguous=False)
        if t.stride(1) != 1 or (rows > 1 and t.stride(0) < width):
            raise KernelError(f"{name}: rows must be dense and must not overlap")
    _check(_lib().st_activation_multiply(_ptr(out), max(out.stride(0), width), _ptr(a), max(a.stride(0), width),
                                         _ptr(b), max(b.stride(0), width) if b is not None else 0, rows, width,
                                         ACTIVATIONS[activation], code, _stream()))
    return out


def activation(x: torch.Tensor, kind: str, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = act(x) elementwise."""
    return activation_multiply(x, None, kind, out)


def multiply(a: torch.Tensor, b: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = a * b elementwise."""
    return activation_multiply(a, b, "none", out)


# ------------------------------------------------- short convolution over time
def _d_token_conv(x, weight, state, ctx_arrays, out_dtype, **kw):
    n, c = x.shape
    return {"rows": n, "width": c, "bytes": n * c * (x.element_size() + torch.empty((), dtype=out_dtype).element_size())}


def _slot_rows(state: torch.Tensor, name: str, inner: int) -> int:
    """``state`` is [slots, ...] float with dense trailing dimensions of ``inner`` elements a slot (a whole
    per-slot tensor, or a part of a larger one): the elements between slots."""
    _need(state, name, torch.float32, contiguous=False)
    if state[0].numel() != inner or not state[0].is_contiguous():
        raise KernelError(f"{name}: a slot must hold {inner} dense floats")
    return state.stride(0) if state.shape[0] > 1 else inner


@_timed("token_conv", _d_token_conv)
def token_conv(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, ctx_arrays, out_dtype: torch.dtype,
               add_input: bool = True, update_state: bool = True, bias: Optional[torch.Tensor] = None,
               activation: str = "none") -> torch.Tensor:
    """y[t] = act((x[t] if add_input) + bias + sum_j weight[:, j] * x(position of t - taps + 1 + j)) per
    channel, over the rows of a batch: what lies before an item's first row is read from ``state``
    [slots, taps - 1, channels] (float; the slots may be parts of a larger per-slot state), which is then
    moved on by the item's rows.

    x: float or bfloat16 [T, channels] (dense rows, any row stride); weight: float [channels, taps];
    bias: float [channels] or None; ``ctx_arrays``: the batch's (token_item, item_len, item_tok_off,
    item_slot)."""
    token_item, item_len, item_tok_off, item_slot = ctx_arrays
    T, C = x.shape
    taps = weight.shape[1]
    _need(x, "x", None, (T, C), contiguous=False)
    if x.stride(1) != 1:
        raise KernelError("x: rows must be dense")
    _need(weight, "weight", torch.float32, (C, taps))
    if bias is not None:
        _need(bias, "bias", torch.float32, (C,))
    if activation not in ACTIVATIONS:
        raise KernelError(f"the kernels know the activations {sorted(ACTIVATIONS)}, not {activation!r}")
    slot_stride = _slot_rows(state, "state", max(taps - 1, 0) * C) if taps > 1 else 0
    _need(token_item, "token_item", torch.int32, (T,))
    B = item_slot.shape[0]
    for name, v in (("item_len", item_len), ("item_tok_off", item_tok_off), ("item_slot", item_slot)):
        _need(v, name, torch.int32, (B,))
    out = empty((T, C), out_dtype, x.device)
    xs = x.stride(0) if T > 1 else C
    _check(_lib().st_token_conv(_ptr(out), _ptr(x), xs, dtype_code(x.dtype), _ptr(weight), _ptr(bias), _ptr(state),
                                slot_stride, _ptr(token_item), _ptr(item_tok_off), _ptr(item_slot), T, C, taps,
                                int(bool(add_input)), ACTIVATIONS[activation], dtype_code(out_dtype), _stream()))
    if update_state:
        _check(_lib().st_token_conv_state(_ptr(state), slot_stride, _ptr(x), xs, dtype_code(x.dtype), _ptr(item_len),
                                          _ptr(item_tok_off), _ptr(item_slot), B, C, taps, _stream()))
    return out


# ------------------------------------------- rotary positions, one-pool page write
@_timed("rotary", lambda q, k, *a, **kw: {"rows": q.shape[0], "width": q.shape[1] + (k.shape[1] if k is not None else 0),
                                          "bytes": 2 * q.shape[0] * (q.shape[1] + (k.shape[1] if k is not None else 0)) *
                                                   q.element_size()})
def rotary(q: torch.Tensor, k: Optional[torch.Tensor], head_dim: int, freq: torch.Tensor, mult: float,
           positions: torch.Tensor, offset: int = 0, interleaved: bool = False) -> None:
    """In place on q [T, heads * head_dim] and k [T, kv_heads * head_dim] (dense rows, any row stride; k may
    be None): of every head the 2 * len(freq) coordinates from ``offset`` on are turned, coordinate i paired
    with i + len(freq) (``interleaved``: 2i with 2i + 1), by the angle positions[t] * freq[i]; cosine and
    sine are multiplied by ``mult``.  Rows with a negative position are left alone."""
    if k is None:
        k = q[:, :0]
    T = q.shape[0]
    half = freq.shape[0]
    _need(freq, "freq", torch.float32, (half,))
    _need(positions, "positions", torch.int32, (T,))
    for name, t in (("q", q), ("k", k)):
        _need(t, name, q.dtype, (T, t.shape[1]), contiguous=False)
        if t.stride(1) != 1 or t.shape[1] % head_dim:
            raise KernelError(f"{name}: dense rows of whole heads")
    if offset < 0 or offset + 2 * half > head_dim:
        raise KernelError(f"{2 * half} turned coordinates from {offset} on do not fit a head of {head_dim}")
    _check(_lib().st_rotary(_ptr(q), q.stride(0), q.shape[1] // head_dim, _ptr(k) if k.shape[1] else None, k.stride(0),
                            k.shape[1] // head_dim, head_dim, 2 * half, int(offset), int(bool(interleaved)), _ptr(freq),
                            float(mult), _ptr(positions), T, dtype_code(q.dtype), _stream()))


@_timed("paged_write", lambda cache, src, *a, **kw: {"rows": src.shape[0], "width": src.shape[1],
                                                      "bytes": 2 * src.numel() * src.element_size()})
def paged_write(cache: torch.Tensor, src: torch.Tensor, token_item: torch.Tensor, positions: torch.Tensor,
                block_table: torch.Tensor, unit_eps: Optional[float] = None) -> None:
    """Each row of src [T, heads * head_dim] (dense rows, any stride) becomes its token's entry of ``cache``
    [pages, heads, page_size, head_dim]; with ``unit_eps`` every head's vector is divided by its root mean
    square (eps inside the root) on the way, in float."""
    num_pages, heads, ps, hd = cache.shape
    T = src.shape[0]
    _need(cache, "cache", src.dtype, (num_pages, heads, ps, hd), contiguous=False)
    if cache.stride()[1:] != (ps * hd, hd, 1):
        raise KernelError("cache: a page must be contiguous")
    _need(src, "src", None, (T, heads * hd), contiguous=False)
    if src.stride(1) != 1:
        raise KernelError("src: rows must be dense")
    _need(token_item, "token_item", torch.int32, (T,))
    _need(positions, "positions", torch.int32, (T,))
    _need(block_table, "block_table", torch.int32)
    _check(_lib().st_paged_write(_ptr(cache), cache.stride(0), _ptr(src), src.stride(0), _ptr(token_item),
                                 _ptr(positions), _ptr(block_table), block_table.shape[1], ps, T, heads, hd,
                                 int(unit_eps is not None), float(unit_eps or 0.0), dtype_code(src.dtype), _stream()))


@_timed("concat_cast", lambda a, b, dtype: {"rows": a.shape[0], "width": a.shape[1] + b.shape[1],
                                            "bytes": (a.numel() + b.numel()) * (4 + torch.empty((), dtype=dtype).element_size())})
def concat_cast(a: torch.Tensor, b: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """[a | b] row by row in ``dtype``, from float rows."""
    T = a.shape[0]
    _need(a, "a", torch.float32, (T, a.shape[1]))
    _need(b, "b", torch.float32, (T, b.shape[1]))
    out = empty((T, a.shape[1] + b.shape[1]), dtype, a.device)
    _check(_lib().st_concat_cast(_ptr(out), _ptr(a), a.shape[1], _ptr(b), b.shape[1], T, dtype_code(dtype), _stream()))
    return out


# ------------------- attention with coupled heads, a sink and a window
def sink_attention_fits(heads: int, key_dim: int, value_dim: int, mixed: bool) -> bool:
    """Whether ``sink_attention`` takes these sizes (a row's queries and a block's scores live in LDS)."""
    return (heads <= 256 and heads * value_dim <= 8192 and
            int(_lib().st_sink_attention_lds(heads, key_dim, int(mixed))) <= 64 * 1024)


def _d_sink_attention(q, k_cache, v_cache, token_item, positions, block_table, heads, scale, **kw):
    return {"rows": q.shape[0], "heads": heads, "kv_heads": k_cache.shape[1], "head_dim": k_cache.shape[3],
            "value_dim": v_cache.shape[3], "window": kw.get("window", 0), "splits": kw.get("num_splits", 1),
            "elem": k_cache.element_size()}


@_timed("sink_attention", _d_sink_attention)
def sink_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, token_item: torch.Tensor,
                   positions: torch.Tensor, block_table: torch.Tensor, heads: int, scale: float, *,
                   window: int = 0, sink: bool = True, head_mix: Optional[torch.Tensor] = None,
                   num_splits: int = 1, out: Optional[torch.Tensor] = None, keep_first: int = 0) -> torch.Tensor:
    """Each query row attends over its request's cached keys [max(0, p - window + 1), p] (window 0: from
    0) and, with ``keep_first`` > 0, over the keys at positions below ``keep_first`` as well.  Every head's scaled products with a key are mixed over the heads by ``head_mix`` (float
    [heads, heads], row = receiving head; None: no mix) before the softmax; ``sink``: one is added to the
    softmax's denominator.

    q: [T, heads * key_dim] (dense rows, any stride); k_cache [pages, kv_heads, page, key_dim];
    v_cache [pages, kv_heads, page, value_dim].  Returns [T, heads * value_dim]."""
    num_pages, nkv, ps, dk = k_cache.shape
    dv = v_cache.shape[3]
    T = q.shape[0]
    _need(k_cache, "k_cache", q.dtype, (num_pages, nkv, ps, dk), contiguous=False)
    _need(v_cache, "v_cache", q.dtype, (v_cache.shape[0], nkv, ps, dv), contiguous=False)
    if k_cache.stride()[1:] != (ps * dk, dk, 1) or v_cache.stride()[1:] != (ps * dv, dv, 1):
        raise KernelError("a page must be contiguous")
    _need(q, "q", None, (T, heads * dk), contiguous=False)
    if q.stride(1) != 1:
        raise KernelError("q rows must be dense")
    _need(token_item, "token_item", torch.int32, (T,))
    _need(positions, "positions", torch.int32, (T,))
    _need(block_table, "block_table", torch.int32)
    if head_mix is not None:
        _need(head_mix, "head_mix", torch.float32, (heads, heads))
    if out is None:
        out = empty((T, heads * dv), q.dtype, q.device)
    _need(out, "out", q.dtype, (T, heads * dv))
    part_o = part_ml = None
    if num_splits > 1:
        part_o = empty((T, num_splits, heads * dv), torch.float32, q.device)
        part_ml = empty((T, num_splits, heads, 2), torch.float32, q.device)
    _check(_lib().st_sink_attention(_ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(q), q.stride(0), _ptr(k_cache),
                                    k_cache.stride(0), _ptr(v_cache), v_cache.stride(0), _ptr(head_mix),
                                    _ptr(token_item), _ptr(positions), _ptr(block_table), block_table.shape[1], ps, T,
                                    heads, nkv, dk, dv, float(scale), int(window), int(keep_first), int(bool(sink)),
                                    int(num_splits),
                                    dtype_code(q.dtype), _stream()))
    return out


# --------------------------------- recurrences with one decay a head and token
@_timed("recurrence_gates", lambda raw, a_log, bias, heads, mode: {"rows": raw.shape[0], "width": heads,
                                                                      "bytes": 4 * raw.shape[0] * (raw.shape[1] + 2 * heads)})
def recurrence_gates(raw: torch.Tensor, a_log: torch.Tensor, bias: torch.Tensor, heads: int, mode: str):
    """Two float [T, heads] tensors from float logits ``raw`` (dense rows, any stride):
    ``"step"``: raw [T, heads] -> (step = softplus(raw + bias), decay = exp(-exp(a_log) * step));
    ``"write"``: raw [T, 2 * heads] -> (strength = sigmoid(raw[:, :heads]),
    decay = exp(-exp(a_log) * softplus(raw[:, heads:] + bias)))."""
    T = raw.shape[0]
    code = {"step": 0, "write": 1}[mode]
    _need(raw, "raw", torch.float32, (T, heads * (1 + code)), contiguous=False)
    if raw.stride(1) != 1:
        raise KernelError("raw: rows must be dense")
    _need(a_log, "a_log", torch.float32, (heads,))
    _need(bias, "bias", torch.float32, (heads,))
    a = empty((T, heads), torch.float32, raw.device)
    b = empty((T, heads), torch.float32, raw.device)
    _check(_lib().st_recurrence_gates(_ptr(a), _ptr(b), _ptr(raw), raw.stride(0), _ptr(a_log), _ptr(bias), T, heads,
                                      code, _stream()))
    return a, b


@_timed("unit_norm", lambda x, *a, **k: {"rows": x.shape[0], "width": x.shape[1], "bytes": 8 * x.numel()})
def unit_norm(x: torch.Tensor, heads: int, eps: float, scale: float = 1.0) -> torch.Tensor:
    """In place on float x [T, heads * dim] (dense rows, any stride): every head's vector divided by
    sqrt(sum of its squares + eps) and multiplied by ``scale``."""
    T = x.shape[0]
    _need(x, "x", torch.float32, (T, x.shape[1]), contiguous=False)
    if x.stride(1) != 1 or x.shape[1] % heads:
        raise KernelError("x: dense rows of whole heads")
    _check(_lib().st_unit_norm(_ptr(x), x.stride(0), T, heads, x.shape[1] // heads, float(eps), float(scale), _stream()))
    return x


def _d_state_scan(q, k, v, gate_a, gate_b, state, ctx_arrays, heads, mode, skip=None, max_item_rows=0):
    T = q.shape[0]
    vd = v.shape[1] // heads
    kd = state.shape[2]
    return {"rows": T, "heads": heads, "key_dim": kd, "value_dim": vd, "items": ctx_arrays[2].shape[0],
            "flops": (4 if mode == "additive" else 6) * T * heads * kd * vd,
            "bytes": 4 * T * (q.shape[1] + k.shape[1] + 2 * v.shape[1] + 2 * heads) +
                     8 * ctx_arrays[2].shape[0] * heads * kd * vd}


@_timed("state_scan", _d_state_scan)
def state_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate_a: torch.Tensor, gate_b: torch.Tensor,
               state: torch.Tensor, ctx_arrays, heads: int, mode: str, skip: Optional[torch.Tensor] = None,
               max_item_rows: int = 0) -> torch.Tensor:
    """Per item and head, from the slot's state S [key_dim, value_dim] and over the item's rows in order
    (a = gate_a[t, head], b = gate_b[t, head]):
    ``"additive"``: S <- b S + (a k_t) v_t^T, o_t = S^T q_t + skip[head] v_t;
    ``"delta"``: S <- b S, u = a (v_t - S^T k_t), S <- S + k_t u^T, o_t = S^T q_t.
    The state is stored back.  q, k: float [T, qk_heads * key_dim], v: float [T, heads * value_dim] (dense
    rows, any stride; head h reads q/k head h // (heads / qk_heads)); state: float
    [slots, heads, key_dim, value_dim] (slots may be parts of a larger per-slot state).  ``max_item_rows``: a
    bound on the rows of any item where the caller knows one (1 in steps of single tokens; 0: the launch's
    rows); it sizes the kernel's staging, nothing else.  Returns float [T, heads * value_dim]."""
    _token_item, item_len, item_tok_off, item_slot = ctx_arrays
    T = q.shape[0]
    _, sh, kd, vd = state.shape
    if sh != heads or v.shape[1] != heads * vd or q.shape[1] % kd or q.shape[1] != k.shape[1]:
        raise KernelError("state_scan: the operands' sizes do not fit the state")
    qk_heads = q.shape[1] // kd
    if heads % qk_heads:
        raise KernelError(f"{heads} heads do not divide over {qk_heads} query/key heads")
    for name, t in (("q", q), ("k", k), ("v", v)):
        _need(t, name, torch.float32, (T, t.shape[1]), contiguous=False)
        if t.stride(1) != 1:
            raise KernelError(f"{name}: rows must be dense")
    # one row of gates serves every token (constants a head), or a row a token
    gate_rows = gate_a.shape[0]
    if gate_rows not in (1, T) and T > 0:
        raise KernelError(f"state_scan: gates for 1 or {T} rows, not {gate_rows}")
    _need(gate_a, "gate_a", torch.float32, (gate_rows, heads))
    _need(gate_b, "gate_b", torch.float32, (gate_rows, heads))
    gate_stride = 0 if gate_rows == 1 else heads
    if skip is not None:
        _need(skip, "skip", torch.float32, (heads,))
    slot_stride = _slot_rows(state, "state", heads * kd * vd)
    B = item_slot.shape[0]
    for name, t in (("item_len", item_len), ("item_tok_off", item_tok_off), ("item_slot", item_slot)):
        _need(t, name, torch.int32, (B,))
    out = empty((T, heads * vd), torch.float32, q.device)
    _check(_lib().st_state_scan(_ptr(out), _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0),
                                _ptr(gate_a), _ptr(gate_b), gate_stride, _ptr(skip), _ptr(state), slot_stride, _ptr(item_len),
                                _ptr(item_tok_off), _ptr(item_slot), B, int(max_item_rows) or T, heads, qk_heads, kd, vd,
                                {"additive": 0, "delta": 1}[mode], _stream()))
    return out


@_timed("retention_chunks", lambda q, k, v, decay, key_factor, state, ctx_arrays, heads: {
    "rows": q.shape[0], "heads": heads, "key_dim": state.shape[2], "value_dim": state.shape[3],
    "items": ctx_arrays[3].shape[0],
    "bytes": 4 * (q.shape[0] * (q.shape[1] + k.shape[1] + 2 * v.shape[1]) +
                  3 * (q.shape[0] // 16 + 1) * heads * state.shape[2] * state.shape[3])})
def retention_chunks(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, key_factor: float,
                     state: torch.Tensor, ctx_arrays, heads: int) -> torch.Tensor:
    """Per item and head, from the slot's state S [key_dim, value_dim] and over the item's rows in order:
    S <- decay[head] S + (key_factor k_t) v_t^T, o_t = S^T q_t; the state is stored back.  What ``state_scan``
    computes in its additive form with constant gates, as products within chunks of rows and a carry between
    chunks: for steps with prompts or portions.  q, k: float [T, heads * key_dim], v: float [T, heads * value_dim]
    (dense rows, any stride); decay: float [heads]; state: float [slots, heads, key_dim, value_dim].  Returns
    float [T, heads * value_dim]; rows of no item are left as they are."""
    _token_item, item_len, item_tok_off, item_slot = ctx_arrays
    T = q.shape[0]
    _, sh, kd, vd = state.shape
    if sh != heads or q.shape[1] != heads * kd or k.shape[1] != heads * kd or v.shape[1] != heads * vd:
        raise KernelError("retention_chunks: the operands' sizes do not fit the state")
    if kd > 256:
        raise KernelError(f"retention_chunks: up to 256 key channels a head, not {kd}")
    for name, t in (("q", q), ("k", k), ("v", v)):
        _need(t, name, torch.float32, (T, t.shape[1]), contiguous=False)
        if t.stride(1) != 1:
            raise KernelError(f"{name}: rows must be dense")
    _need(decay, "decay", torch.float32, (heads,))
    slot_stride = _slot_rows(state, "state", heads * kd * vd)
    B = item_slot.shape[0]
    for name, t in (("item_len", item_len), ("item_tok_off", item_tok_off), ("item_slot", item_slot)):
        _need(t, name, torch.int32, (B,))
    out = empty((T, heads * vd), torch.float32, q.device)
    chunks = T // int(_lib().st_retention_chunk_rows(kd)) + B
    scratch = empty((max(chunks, 1), heads, kd, vd), torch.float32, q.device)
    _check(_lib().st_retention_chunks(_ptr(out), _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0),
                                      _ptr(decay), float(key_factor), _ptr(state), slot_stride, _ptr(item_len),
                                      _ptr(item_tok_off), _ptr(item_slot), B, T, heads, kd, vd, _ptr(scratch), chunks,
                                      _stream()))
    return out


@_timed("gated_group_norm", lambda o, gate, *a, **k: {"rows": o.shape[0], "width": o.shape[1],
                                                       "bytes": o.numel() * (4 + 3 * gate.element_size())})
def gated_group_norm(o: torch.Tensor, gate: torch.Tensor, gain: torch.Tensor, groups: int, eps: float,
                     out_dtype: torch.dtype, gate_first: bool = False, gate_kind: str = "silu") -> torch.Tensor:
    """Each of the ``groups`` equal parts of a row of o (float [T, W]) divided by its root mean square and
    multiplied by ``gain`` (float [W / groups] shared by the parts, or [W]) and by silu(gate) (``gate``:
    [T, W] rows of ``out_dtype``, any stride); ``gate_first``: the gate multiplies before the norm;
    ``gate_kind`` "sigmoid": sigmoid(gate) in silu's place."""
    if gate_kind not in ("silu", "sigmoid"):
        raise KernelError(f"the gate is silu or sigmoid, not {gate_kind!r}")
    T, W = o.shape
    if W % groups:
        raise KernelError(f"{W} channels do not divide into {groups} parts")
    width = W // groups
    _need(o, "o", torch.float32, (T, W))
    _need(gate, "gate", out_dtype, (T, W), contiguous=False)
    if gate.stride(1) != 1:
        raise KernelError("gate: rows must be dense")
    if tuple(gain.shape) not in ((width,), (W,)):
        raise KernelError(f"gain must have {width} or {W} entries")
    _need(gain, "gain", torch.float32)
    out = empty((T, W), out_dtype, o.device)
    _check(_lib().st_gated_group_norm(_ptr(out), _ptr(o), _ptr(gate), gate.stride(0), _ptr(gain), T, groups, width,
                                      int(gain.shape[0] == W and groups > 1), int(bool(gate_first)),
                                      int(gate_kind == "sigmoid"), float(eps),
                                      dtype_code(out_dtype), _stream()))
    return out


# ------------------------------------------------------ gated linear attention
@_timed("decay_gate", lambda z, inv_tau, out=None: {"rows": z.shape[0], "width": z.shape[-1], "bytes": 8 * z.numel()})
def decay_gate(z: torch.Tensor, inv_tau: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """sigmoid(z) ** inv_tau (float), computed as exp(inv_tau * log sigmoid(z)); in place unless ``out``."""
    _need(z, "z", torch.float32)
    if out is None:
        out = z
    _need(out, "out", torch.float32, z.shape)
    _check(_lib().st_decay_gate(_ptr(out), _ptr(z), z.numel(), float(inv_tau), _stream()))
    return out


class PartialSums:
    """A result still split into planes that are to be summed: ``planes`` float [parts, T, width]."""

    def __init__(self, planes: torch.Tensor):
        self.planes = planes

    def sum(self) -> torch.Tensor:
        return self.planes.sum(0)


def _d_gla_scan(q, k, v, decay, state, ctx_arrays, heads, scale, part_dim=0):
    T = q.shape[0]
    kd, vd = q.shape[1] // heads, v.shape[1] // heads
    parts = -(-kd // (part_dim or 16))
    return {"rows": T, "heads": heads, "key_dim": kd, "value_dim": vd, "items": ctx_arrays[2].shape[0], "parts": parts,
            "flops": 4 * T * heads * kd * vd,
            # operands of every row, the planes of partial results, and the items' states read and written once
            "bytes": T * heads * ((2 * kd + vd) * q.element_size() + 4 * kd + 4 * vd * parts) +
                     8 * ctx_arrays[2].shape[0] * heads * kd * vd}


@_timed("gla_scan", _d_gla_scan)
def gla_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, state: torch.Tensor,
             ctx_arrays, heads: int, scale: float, part_dim: int = 0) -> PartialSums:
    """Per item and head, from the slot's state S and over the item's rows in order:
    S <- diag(decay_t) S + k_t v_t^T, o_t = scale * S^T q_t; the state is stored back.

    q, k: [T, heads * key_dim], v: [T, heads * value_dim] views (dense rows, any row stride);
    decay: float [T, heads * key_dim]; state: float [slots, heads, key_dim, value_dim].  The key
    channels are dealt to parts of ``part_dim`` (4, 8 or 16; 0: 16); the result
    comes as the parts' planes [parts, T, heads * value_dim], whose sum is o (``gated_head_norm``
    sums them)."""
    _token_item, item_len, item_tok_off, item_slot = ctx_arrays
    T = q.shape[0]
    kd, vd = q.shape[1] // heads, v.shape[1] // heads
    for name, t, w in (("q", q, heads * kd), ("k", k, heads * kd), ("v", v, heads * vd)):
        _need(t, name, q.dtype, (T, w), contiguous=False)
        if t.stride(1) != 1:
            raise KernelError(f"{name}: rows must be dense")
    _need(decay, "decay", torch.float32, (T, heads * kd))
    _need(state, "state", torch.float32, (state.shape[0], heads, kd, vd))
    B = item_slot.shape[0]
    for name, t in (("item_len", item_len), ("item_tok_off", item_tok_off), ("item_slot", item_slot)):
        _need(t, name, torch.int32, (B,))
    part_dim = int(part_dim) or 16
    parts = -(-kd // part_dim)
    planes = empty((parts, T, heads * vd), torch.float32, q.device)
    _check(_lib().st_gla_scan(_ptr(planes), T * heads * vd, part_dim, _ptr(q), q.stride(0), _ptr(k), k.stride(0),
                              _ptr(v), v.stride(0), _ptr(decay), _ptr(state), _ptr(item_len), _ptr(item_tok_off),
                              _ptr(item_slot), B, heads, kd, vd, float(scale), dtype_code(q.dtype), _stream()))
    return PartialSums(planes)


@_timed("gated_head_norm", lambda o, gate, *a, **k: {
    "rows": gate.shape[0], "width": gate.shape[1],
    "bytes": gate.numel() * (2 * gate.element_size() + 4 * (o.planes.shape[0] if isinstance(o, PartialSums) else 1))})
def gated_head_norm(o, gate: torch.Tensor, gain: torch.Tensor, heads: int, eps: float,
                    out_dtype: torch.dtype) -> torch.Tensor:
    """out[t, h, :] = o[t, h, :] * rsqrt(mean(o[t, h, :]^2) + eps) * gain * silu(gate[t, h, :]).
    o: float [T, heads * value_dim], or the ``PartialSums`` whose planes sum to it; gate: a view of
    ``out_dtype`` rows; gain: float [value_dim]."""
    planes = o.planes if isinstance(o, PartialSums) else o.unsqueeze(0)
    parts, T, width = planes.shape
    vd = width // heads
    _need(planes, "o", torch.float32, (parts, T, heads * vd))
    _need(gate, "gate", out_dtype, (T, heads * vd), contiguous=False)
    if gate.stride(1) != 1:
        raise KernelError("gate: rows must be dense")
    _need(gain, "gain", torch.float32, (vd,))
    out = empty((T, heads * vd), out_dtype, planes.device)
    _check(_lib().st_gated_head_norm(_ptr(out), _ptr(planes), parts, T * width, _ptr(gate), gate.stride(0),
                                     _ptr(gain), T, heads, vd, float(eps), dtype_code(out_dtype), _stream()))
    return out


# ------------------------------------------------------------------ latent cache
@_timed("latent_write", lambda cache, x, *a, **k: {"rows": x.shape[0], "width": x.shape[1],
                                                   "bytes": x.numel() * (4 + cache.element_size())})
def latent_write(cache: torch.Tensor, x: torch.Tensor, gain: torch.Tensor, eps: float, token_item: torch.Tensor,
                 positions: torch.Tensor, block_table: torch.Tensor, tail: int = 0,
                 tail_freq: Optional[torch.Tensor] = None, tail_mult: float = 1.0) -> None:
    """Each row of x (float [T, rank + tail], dense rows of any stride): its first ``rank`` values are
    normalised to unit root mean square, multiplied by ``gain`` and stored as its token's entry of ``cache``
    [pages, 1, page_size, entry] with entry >= rank + tail; the ``tail`` values after them follow in the
    entry as they are, or, with ``tail_freq`` (float [tail / 2]), turned by the token's position (pairs
    2i, 2i + 1; angle position * tail_freq[i]; cosine and sine times ``tail_mult``); the rest of an entry is
    cleared."""
    num_pages, one, ps, entry = cache.shape
    T = x.shape[0]
    rank = x.shape[1] - int(tail)
    _need(cache, "cache", None, (num_pages, 1, ps, entry), contiguous=False)
    if rank <= 0 or cache.stride()[1:] != (ps * entry, entry, 1) or entry < rank + tail:
        raise KernelError("latent_write: pages of one head must be contiguous and an entry as wide as the row")
    if tail_freq is not None:
        _need(tail_freq, "tail_freq", torch.float32, (tail // 2,))
        if tail % 2:
            raise KernelError("latent_write: a turned tail has an even size")
    _need(x, "x", torch.float32, (T, rank + tail), contiguous=False)
    if x.stride(1) != 1:
        raise KernelError("x: rows must be dense")
    _need(gain, "gain", torch.float32, (rank,))
    _need(token_item, "token_item", torch.int32, (T,))
    _need(positions, "positions", torch.int32, (T,))
    _need(block_table, "block_table", torch.int32)
    _check(_lib().st_latent_write(_ptr(cache), cache.stride(0), _ptr(x), x.stride(0), _ptr(gain), _ptr(token_item),
                                  _ptr(positions), _ptr(block_table), block_table.shape[1], ps, T, rank, entry,
                                  float(eps), int(tail), _ptr(tail_freq), float(tail_mult), dtype_code(cache.dtype),
                                  _stream()))


# ---------------------------------------------------------------- routed experts
def moe_tile(num_tokens: int, top: int, experts: int) -> int:
    """Places a tile: 16 for few rows an expert (only the weights' stream counts), 64 or 128 where an
    expert gets some dozens or a hundred rows on average (a tile's weight operands then meet four or
    eight blocks of 16 rows, and the expert's weights are read once a tile)."""
    pairs = num_tokens * top
    return 128 if pairs >= 96 * experts else 64 if pairs >= 32 * experts else 16


def moe_capacity(num_tokens: int, top: int, experts: int, tile: int) -> int:
    """Places of the sorted pair list: every expert's pairs start a tile of their own."""
    return -(-num_tokens * top // tile) * tile + tile * experts


def _d_moe(x, logits, w_gate, w_up, w_down, residual, *, top, limit=0.0, out_scale=1.0, token_item=None, **kw):
    T, W = x.shape
    E, F, _ = w_gate.shape
    used = min(E, T * top)
    return {"rows": T, "width": W, "inner": F, "experts": E, "top": top,
            "flops": 6 * T * top * W * F, "bytes": used * 3 * F * W * x.element_size() + T * W * (x.element_size() + 8)}


@_timed("routed_experts", _d_moe)
def routed_experts(x: torch.Tensor, logits: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor,
                   w_down: torch.Tensor, residual: Optional[torch.Tensor], *, top: int, limit: float = 0.0,
                   out_scale: float = 1.0, token_item: Optional[torch.Tensor] = None,
                   style: str = "scaled_input", groups: int = 1, keep: int = 1) -> torch.Tensor:
    """residual <- residual + out_scale * sum over a row's ``top`` best experts e (by ``logits``) of
    Wd[e] y with y = g * sigmoid(1.702 g) * (u + 1), g = min(s * Wg[e] x, limit),
    u = clamp(s * Wu[e] x, -limit, limit), s = sigmoid(logit of e).  In place on ``residual``
    (float [T, width]), which is returned.

    ``style`` "softmax_output": the weights of a row's experts are the softmax over their logits alone and
    multiply the experts' results, sum_e s_e Wd[e] (silu(Wg[e] x) * (Wu[e] x)), with no limit.  Then
    ``residual`` may be None: the weighted sum itself is returned (a new float tensor).
    ``style`` "softmax_all": the same experts, weighted by their shares of the softmax over all experts' logits
    (not renormalised); only experts of the ``keep`` best of ``groups`` equal groups of neighbours can be chosen,
    a group ranking by its largest logit.

    x: [T, width]; logits: float [T, experts]; w_gate, w_up: [experts, inner, width]; w_down:
    [experts, width, inner].  Rows whose ``token_item`` is negative are left as they are."""
    T, W = x.shape
    E, F, _ = w_gate.shape
    _need(x, "x", w_gate.dtype, (T, W))
    _need(logits, "logits", torch.float32, (T, E))
    _need(w_gate, "w_gate", None, (E, F, W))
    _need(w_up, "w_up", w_gate.dtype, (E, F, W))
    _need(w_down, "w_down", w_gate.dtype, (E, W, F))
    if style not in ("scaled_input", "softmax_output", "softmax_all"):
        raise KernelError(f"routed_experts: unknown style {style!r}")
    on_output = style != "scaled_input"
    mode = {"scaled_input": 0, "softmax_output": 1, "softmax_all": 2}[style]
    if mode == 2 and (groups < 1 or E % groups or not 1 <= keep <= groups or top > keep * (E // groups)):
        raise KernelError(f"routed_experts: {top} of {E} experts in {groups} groups of which {keep} are kept")
    if residual is None and not on_output:
        raise KernelError("routed_experts: this style adds to a residual stream")
    if residual is not None:
        _need(residual, "residual", torch.float32, (T, W))
    if token_item is not None:
        _need(token_item, "token_item", torch.int32, (T,))
    lib, dev, code, st = _lib(), x.device, dtype_code(x.dtype), _stream()
    tile = moe_tile(T, top, E)
    cap = moe_capacity(T, top, E, tile)
    ids = empty((T * top,), torch.int32, dev)
    wts = empty((T * top,), torch.float32, dev)
    sorted_pairs = empty((cap,), torch.int32, dev)
    place = empty((T * top,), torch.int32, dev)
    tile_expert = empty((cap // tile,), torch.int32, dev)
    y = empty((cap, F), x.dtype, dev)
    _check(lib.st_moe_route(_ptr(ids), _ptr(wts), _ptr(logits), _ptr(token_item), T, E, int(top), mode, int(groups), int(keep), st))
    _check(lib.st_moe_align(_ptr(sorted_pairs), _ptr(place), _ptr(tile_expert), _ptr(ids), T * top, E, cap, tile, st))
    _check(lib.st_moe_up(_ptr(y), _ptr(x), _ptr(w_gate), _ptr(w_up), _ptr(sorted_pairs), _ptr(tile_expert),
                         _ptr(wts), cap, tile, int(top), W, F, float(limit), int(on_output), code, st))
    if on_output:
        out = residual if residual is not None else empty((T, W), torch.float32, dev)
        pair_out = empty((cap, W), torch.float32, dev)
        _check(lib.st_moe_down(None, None, _ptr(pair_out), _ptr(y), _ptr(w_down), _ptr(sorted_pairs),
                               _ptr(tile_expert), cap, tile, int(top), W, F, 1.0, code, st))
        _check(lib.st_moe_combine(_ptr(out), _ptr(residual), _ptr(pair_out), _ptr(place), _ptr(wts), T, int(top), W,
                                  float(out_scale), st))
        return out
    if top == 1:
        _check(lib.st_moe_down(_ptr(residual), _ptr(residual), None, _ptr(y), _ptr(w_down), _ptr(sorted_pairs),
                               _ptr(tile_expert), cap, tile, 1, W, F, float(out_scale), code, st))
    else:
        pair_out = empty((cap, W), torch.float32, dev)
        _check(lib.st_moe_down(None, None, _ptr(pair_out), _ptr(y), _ptr(w_down), _ptr(sorted_pairs),
                               _ptr(tile_expert), cap, tile, int(top), W, F, float(out_scale), code, st))
        _check(lib.st_moe_combine(_ptr(residual), _ptr(residual), _ptr(pair_out), _ptr(place), None, T, int(top), W,
                                  float(out_scale), st))
    return residual


# -------------------------------------------- float operations on the residual stream
@_timed("dynamic_tanh", lambda x, *a, **k: {"rows": (k.get("rows").shape[0] if k.get("rows") is not None else x.shape[0]),
                                            "width": x.shape[1], "bytes": 10 * x.shape[1] *
                                            (k.get("rows").shape[0] if k.get("rows") is not None else x.shape[0])})
def dynamic_tanh(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], alpha: torch.Tensor, *,
                 rows: Optional[torch.Tensor] = None, out_t: Optional[torch.Tensor] = None,
                 out_f32: Optional[torch.Tensor] = None, base: Optional[torch.Tensor] = None,
                 then: Optional[tuple] = None) -> None:
    """y = tanh(alpha * x) * weight + bias per element of the float rows x [T, width] (of the rows picked by
    ``rows``, int32, negative entries skipped); ``alpha``: float [1] on the device.  ``base`` (float, the
    result's shape): y += base.  Written to ``out_f32`` (float) and / or ``out_t`` (float or bfloat16).
    ``then`` = (weight2, bias2 or None, alpha2): ``out_t`` receives tanh(alpha2 * y) * weight2 + bias2
    instead of y (``out_f32`` still y)."""
    T, W = x.shape
    n = rows.shape[0] if rows is not None else T
    _need(x, "x", torch.float32, (T, W))
    _need(weight, "weight", torch.float32, (W,))
    if bias is not None:
        _need(bias, "bias", torch.float32, (W,))
    _need(alpha, "alpha", torch.float32, (1,))
    if rows is not None:
        _need(rows, "rows", torch.int32, (n,))
    if out_t is None and out_f32 is None:
        raise KernelError("dynamic_tanh: no output")
    if out_f32 is not None:
        _need(out_f32, "out_f32", torch.float32, (n, W))
    if out_t is not None:
        _need(out_t, "out_t", None, (n, W))
    if base is not None:
        _need(base, "base", torch.float32, (n, W))
    w2 = b2 = a2 = None
    if then is not None:
        w2, b2, a2 = then
        _need(w2, "weight2", torch.float32, (W,))
        if b2 is not None:
            _need(b2, "bias2", torch.float32, (W,))
        _need(a2, "alpha2", torch.float32, (1,))
        if out_t is None:
            raise KernelError("dynamic_tanh: the second norm goes to out_t")
    _check(_lib().st_dynamic_tanh(_ptr(out_t), _ptr(out_f32), _ptr(x), _ptr(rows), _ptr(weight), _ptr(bias), _ptr(alpha),
                                  _ptr(base), _ptr(w2), _ptr(b2), _ptr(a2), n, W,
                                  dtype_code(out_t.dtype) if out_t is not None else F32, _stream()))


@_timed("unit_add", lambda x, y, *a, **k: {"rows": x.shape[0], "width": x.shape[1], "bytes": 12 * x.numel()})
def unit_add(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x += y / sqrt(mean(y^2) + eps) * weight row by row, in place on the float rows x [T, width]."""
    T, W = x.shape
    _need(x, "x", torch.float32, (T, W))
    _need(y, "y", torch.float32, (T, W))
    _need(weight, "weight", torch.float32, (W,))
    _check(_lib().st_unit_add(_ptr(x), _ptr(y), _ptr(weight), T, W, float(eps), _stream()))
    return x


def token_side_fits(width: int, dim: int) -> bool:
    """Whether ``token_side`` takes these sizes: a row and the gated vector as floats in 60 KB of LDS."""
    return 4 * (width + dim) <= 60 * 1024


@_timed("token_side", lambda x, ids, item, table, w_gate, *a, **k: {
    "rows": x.shape[0], "width": x.shape[1], "inner": w_gate.shape[0],
    "bytes": 8 * x.numel() + 2 * w_gate.numel() * w_gate.element_size()})
def token_side(x: torch.Tensor, token_ids: torch.Tensor, token_item: Optional[torch.Tensor], table: torch.Tensor,
               w_gate: torch.Tensor, w_proj: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """x[t] += unit(w_proj (gelu_tanh(w_gate x[t]) * table[token_ids[t]])) * gain, in place on the float rows x
    [T, width]; unit(y) = y / sqrt(mean(y^2) + eps).  table [vocab, dim] (rows may be strided: columns of a wider
    table), w_gate [dim, width], w_proj [width, dim] of one storage type; the row, the sums and the gated vector are
    float.  Rows with token_item < 0 are left alone."""
    T, W = x.shape
    dim = w_gate.shape[0]
    _need(x, "x", torch.float32, (T, W))
    _need(token_ids, "token_ids", torch.int32, (T,))
    if token_item is not None:
        _need(token_item, "token_item", torch.int32, (T,))
    dt = w_gate.dtype
    _need(w_gate, "w_gate", dt, (dim, W))
    _need(w_proj, "w_proj", dt, (W, dim))
    _need(table, "table", dt, (table.shape[0], dim), contiguous=False)
    if table.stride(1) != 1:
        raise KernelError("table: rows must be dense")
    _need(gain, "gain", torch.float32, (W,))
    if not token_side_fits(W, dim):
        raise KernelError(f"token_side: a row of {W} and a gated vector of {dim} do not fit the LDS")
    _check(_lib().st_token_side(_ptr(x), _ptr(token_ids), _ptr(token_item), _ptr(table), table.stride(0), table.shape[0],
                                _ptr(w_gate), _ptr(w_proj), _ptr(gain), T, dim, W, float(eps), dtype_code(dt), _stream()))
    return x


@_timed("row_add", lambda x, *a, **k: {"rows": x.shape[0], "width": x.shape[1], "bytes": 12 * x.numel()})
def row_add(x: torch.Tensor, first: Optional[torch.Tensor], vec: torch.Tensor) -> torch.Tensor:
    """x (+ first) + vec: float rows [T, width], a second stream of the same shape or None, and one float
    vector [width] for every row.  Returns a new tensor."""
    T, W = x.shape
    _need(x, "x", torch.float32, (T, W))
    if first is not None:
        _need(first, "first", torch.float32, (T, W))
    _need(vec, "vec", torch.float32, (W,))
    out = empty((T, W), torch.float32, x.device)
    _check(_lib().st_row_add(_ptr(out), _ptr(x), _ptr(first), _ptr(vec), T, W, _stream()))
    return out


@_timed("scale_softcap", lambda x, *a, **k: {"rows": x.shape[0], "width": x.shape[-1], "bytes": 8 * x.numel()})
def scale_softcap(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """x <- cap * tanh(x * scale / cap) (``cap`` <= 0: x * scale), in place on a dense float tensor."""
    _need(x, "x", torch.float32)
    _check(_lib().st_scale_softcap(_ptr(x), x.numel(), float(scale), float(cap), _stream()))
    return x


# ------------------------------------------------ a residual stream of several copies
@_timed("streams_expand", lambda x, streams: {"rows": x.shape[0], "width": x.shape[1], "bytes": 4 * x.numel() * (1 + streams)})
def streams_expand(x: torch.Tensor, streams: int) -> torch.Tensor:
    """[T, W] float -> [T, streams * W]: every stream a copy of the row."""
    T, W = x.shape
    _need(x, "x", torch.float32, (T, W))
    out = empty((T, streams * W), torch.float32, x.device)
    _check(_lib().st_streams_expand(_ptr(out), _ptr(x), T, int(streams), W, _stream()))
    return out


def streams_sum(x: torch.Tensor, streams: int, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The sum of the streams of x (float [T, streams * W]) for every row, or for the rows picked by ``rows``
    (int32; a negative entry gives zeros): float [rows, W]."""
    T, SW = x.shape
    if SW % streams:
        raise KernelError(f"{SW} columns are not {streams} streams")
    W = SW // streams
    _need(x, "x", torch.float32, (T, SW))
    n = T
    if rows is not None:
        n = rows.shape[0]
        _need(rows, "rows", torch.int32, (n,))
    out = empty((n, W), torch.float32, x.device)
    _check(_lib().st_streams_sum(_ptr(out), _ptr(x), _ptr(rows), n, int(streams), W, _stream()))
    return out


@_timed("streams_read", lambda x, weights, *a, **k: {"rows": x.shape[0], "width": x.shape[1],
                                                     "bytes": x.numel() * 4 + x.numel() // weights.shape[0] * 2})
def streams_read(x: torch.Tensor, weights: torch.Tensor, gain: Optional[torch.Tensor], eps: float,
                 out_dtype: torch.dtype) -> torch.Tensor:
    """u = sum_s weights[s] x_s of the streams x (float [T, S * W]), then u * rsqrt(mean(u^2) + eps) * gain
    (``eps`` <= 0: u itself) in ``out_dtype``: what a sublayer reads."""
    T, SW = x.shape
    S = weights.shape[0]
    W = SW // S
    _need(x, "x", torch.float32, (T, S * W))
    _need(weights, "weights", torch.float32, (S,))
    if gain is not None:
        _need(gain, "gain", torch.float32, (W,))
    out = empty((T, W), out_dtype, x.device)
    _check(_lib().st_streams_read(_ptr(out), None, _ptr(x), _ptr(weights), _ptr(gain), T, S, W, float(eps),
                                  dtype_code(out_dtype), _stream()))
    return out


@_timed("streams_write", lambda x, y, mix, *a, **k: {"rows": x.shape[0], "width": x.shape[1],
                                                     "bytes": x.numel() * 8 + y.numel() * 4})
def streams_write(x: torch.Tensor, y: torch.Tensor, mix: torch.Tensor, out_weights: torch.Tensor,
                  then: Optional[tuple] = None, out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """In place on the streams x (float [T, S * W]): x_t <- sum_s mix[s, t] x_s + out_weights[t] * y, y float
    [T, W].  ``then`` = (weights, gain or None, eps): also returns the next sublayer's read of the new streams
    (as ``streams_read``) in ``out_dtype``, made in the same pass."""
    T, SW = x.shape
    S = out_weights.shape[0]
    W = SW // S
    _need(x, "x", torch.float32, (T, S * W))
    _need(y, "y", torch.float32, (T, W))
    _need(mix, "mix", torch.float32, (S, S))
    _need(out_weights, "out_weights", torch.float32, (S,))
    nxt = a2 = g2 = None
    eps2, code = 0.0, F32
    if then is not None:
        a2, g2, eps2 = then
        _need(a2, "next weights", torch.float32, (S,))
        if g2 is not None:
            _need(g2, "next gain", torch.float32, (W,))
        nxt = empty((T, W), out_dtype, x.device)
        code = dtype_code(out_dtype)
    _check(_lib().st_streams_write(_ptr(x), _ptr(y), _ptr(mix), _ptr(out_weights), _ptr(nxt), _ptr(a2), _ptr(g2), T, S,
                                   W, float(eps2), code, _stream()))
    return nxt


@_timed("hashed_embed", lambda ids, positions, ctx_arrays, last_token, table, pairs, *a, **k: {
    "rows": ids.shape[0], "width": table.shape[1],
    "bytes": ids.shape[0] * table.shape[1] * (4 + table.element_size() * (2 if pairs is not None else 1))})
def hashed_embed(ids: torch.Tensor, positions: torch.Tensor, ctx_arrays, last_token: Optional[torch.Tensor],
                 table: torch.Tensor, pairs: Optional[torch.Tensor], mul_prev: int, mul_cur: int,
                 scale: float) -> torch.Tensor:
    """x[t] = table[id_t] * scale + pairs[(id_(t-1) * mul_prev + id_t * mul_cur) mod buckets], float [T, W];
    pairs [buckets + 1, W], its last row for a sequence's first token.  ``ctx_arrays`` = (token_item, item_len,
    item_tok_off, item_slot); ``last_token`` (int32 [slots]): the last token of each slot's request so far,
    read for an item's first row and moved on to the item's last token of this step.  ``pairs`` None: the
    token's row times the factor alone."""
    token_item, item_len, item_tok_off, item_slot = ctx_arrays
    T = ids.shape[0]
    V, W = table.shape
    _need(table, "table", None, (V, W))
    buckets = 0
    if pairs is not None:
        _need(pairs, "pairs", table.dtype, (pairs.shape[0], W))
        if pairs.shape[0] < 2:
            raise KernelError("the table of pairs has a row a bucket and one more")
        buckets = pairs.shape[0] - 1
        _need(last_token, "last_token", torch.int32)
    for name, v in (("ids", ids), ("positions", positions), ("token_item", token_item)):
        _need(v, name, torch.int32, (T,))
    B = item_len.shape[0]
    for name, v in (("item_len", item_len), ("item_tok_off", item_tok_off), ("item_slot", item_slot)):
        _need(v, name, torch.int32, (B,))
    out = empty((T, W), torch.float32, table.device)
    _check(_lib().st_hashed_embed(_ptr(out), _ptr(ids), _ptr(positions), _ptr(token_item), _ptr(item_len),
                                  _ptr(item_tok_off), _ptr(item_slot), _ptr(last_token), _ptr(table), _ptr(pairs), T, B,
                                  V, buckets, int(mul_prev), int(mul_cur), float(scale), W,
                                  dtype_code(table.dtype), _stream()))
    return out


@_timed("qk_norm_write", lambda qk, gain_q, gain_k, eps, heads, kv_heads, head_dim, k_cache, *a, **k: {
    "rows": qk.shape[0], "width": qk.shape[1],
    "bytes": qk.shape[0] * (4 * qk.shape[1] + k_cache.element_size() * k_cache.shape[3] * (heads + 2 * kv_heads))})
def qk_norm_write(qk: torch.Tensor, gain_q: torch.Tensor, gain_k: torch.Tensor, eps: float, heads: int, kv_heads: int,
                  head_dim: int, k_cache: torch.Tensor, v_cache: torch.Tensor, token_item: torch.Tensor,
                  positions: torch.Tensor, block_table: torch.Tensor, write: bool = True) -> torch.Tensor:
    """qk: float [T, (heads + kv_heads) * head_dim], queries then keys.  Both are divided by their root mean
    square over the whole projection and multiplied by their gains; returns the queries [T, heads * head_pad]
    in the pools' type (head_pad: the pools' entry width, zeros behind head_dim) and, with ``write``, stores
    the normalised keys in ``k_cache`` and the keys as projected in ``v_cache``."""
    num_pages, nkv, ps, pad = k_cache.shape
    T = qk.shape[0]
    _need(qk, "qk", torch.float32, (T, (heads + kv_heads) * head_dim), contiguous=False)
    if qk.stride(1) != 1:
        raise KernelError("qk: rows must be dense")
    if nkv != kv_heads or pad < head_dim or tuple(v_cache.shape) != tuple(k_cache.shape) or \
            k_cache.stride()[1:] != (ps * pad, pad, 1) or v_cache.stride() != k_cache.stride():
        raise KernelError("qk_norm_write: the pools do not fit the keys")
    _need(gain_q, "gain_q", torch.float32, (heads * head_dim,))
    _need(gain_k, "gain_k", torch.float32, (kv_heads * head_dim,))
    _need(token_item, "token_item", torch.int32, (T,))
    _need(positions, "positions", torch.int32, (T,))
    _need(block_table, "block_table", torch.int32)
    out = empty((T, heads * pad), k_cache.dtype, qk.device)
    _check(_lib().st_qk_norm_write(_ptr(out), _ptr(k_cache), _ptr(v_cache), k_cache.stride(0), _ptr(qk), qk.stride(0),
                                   _ptr(gain_q), _ptr(gain_k), _ptr(token_item), _ptr(positions), _ptr(block_table),
                                   block_table.shape[1], ps, T, heads, kv_heads, head_dim, pad, float(eps), int(write),
                                   dtype_code(k_cache.dtype), _stream()))
    return out


def probe_read(src: torch.Tensor, sink: torch.Tensor, workgroups: int, pattern: int = 0) -> None:
    """Measurement aid: a plain read of all of ``src`` by ``workgroups`` workgroups (``sink``: int32,
    one word a workgroup).  ``pattern``: 0 / 1 the grid strides over the buffer with 4 / 8 loads in
    flight per thread, 2 / 3 tiles of 8 / 16 KB dealt round-robin to the workgroups."""
    _need(src, "src")
    _need(sink, "sink", torch.int32)
    nbytes = src.numel() * src.element_size()
    if nbytes % 16 or sink.numel() < workgroups:
        raise KernelError("probe_read: the source must be a multiple of 16 bytes, the sink one word a workgroup")
    _check(_lib().st_probe_read(_ptr(src), nbytes, _ptr(sink), int(workgroups), int(pattern), _stream()))


def probe_empty(sink: torch.Tensor) -> None:
    """Measurement aid: a kernel of one workgroup that does one store."""
    _need(sink, "sink", torch.int32)
    _check(_lib().st_probe_empty(_ptr(sink), _stream()))


def probe_fill(src: torch.Tensor, region: int, sink: torch.Tensor, workgroups: int, turns: int, to_lds: bool) -> None:
    """Measurement aid: ``workgroups`` workgroups each go ``turns`` times 32 KB round their own
    ``region`` bytes of ``src``, by direct loads into LDS or by loads into registers."""
    _need(src, "src")
    _need(sink, "sink", torch.int32)
    if src.numel() * src.element_size() < workgroups * region or sink.numel() < workgroups:
        raise KernelError("probe_fill: the source holds a region a workgroup, the sink one word a workgroup")
    _check(_lib().st_probe_fill(_ptr(src), int(region), _ptr(sink), int(workgroups), int(turns), int(bool(to_lds)),
                                _stream()))


def probe_mfma(sink: torch.Tensor, workgroups: int, rounds: int, wide: bool) -> None:
    """Measurement aid: ``workgroups`` workgroups of four waves issue 16 * ``rounds`` independent
    matrix-core products a wave (bfloat16, the 32x32x16 form if ``wide``, else 16x16x32)."""
    _need(sink, "sink", torch.int32)
    if sink.numel() < workgroups:
        raise KernelError("probe_mfma: the sink holds one word a workgroup")
    _check(_lib().st_probe_mfma(_ptr(sink), int(workgroups), int(rounds), int(bool(wide)), _stream()))


def hash_uniform(seed_lo: int, seed_hi: int, draw: int, v: int) -> float:
    """Host copy of the sampler's counter-based uniform (for plain references)."""
    return float(_lib().st_hash_uniform(seed_lo & 0xffffffff, seed_hi & 0xffffffff,
                                        draw & 0xffffffff, v & 0xffffffff))
