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
    "ms_embed": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "ms_rms_norm": [_c_ptr, _c_ptr, _c_int, _c_int, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int,
                    _c_int, _c_ptr],
    "ms_gemm_skinny_norm": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ll, _c_int,
                            _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_qkv_rope_store": [_c_ptr, _c_ll, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "ms_decode_advance": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
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
                                   _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ll, _c_float, _c_int, _c_int,
                                   _c_int, _c_ptr],
    "ms_attention_mfma_supported": [_c_int, _c_int],
    "ms_paged_attention_mfma": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ll,
                                _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "ms_paged_attention_mfma_decode": [_c_ptr, _c_ll, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                       _c_ll, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                       _c_int, _c_int, _c_int, _c_ptr],
    "ms_argmax": [_c_ptr, _c_ll, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr],
    "ms_sample": [_c_ptr, _c_ll, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                  _c_ptr],
    "ms_sample_workspace_bytes": [_c_int],
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
def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[n] = float(table[ids[n]]).  ids int32 [N] (checked against the table by the caller), out float32 [N, H]."""
    _check(ids, "ids", torch.int32)
    _check(table, "table")
    V, H = table.shape
    _check(out, "out", torch.float32, (ids.numel(), H))
    _call("ms_embed", ids.data_ptr(), table.data_ptr(), out.data_ptr(), ids.numel(), H, _code(table.dtype), _stream())
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
                   page_size: int, draw_index: Optional[torch.Tensor] = None) -> None:
    """Between two decode steps queued back to back: rows below ``n_live[0]`` move one position on, take
    ``prev_tokens`` as their input, count ``draw_index`` up by one and get their new slots from ``tables`` (one
    [table rows, width] per cache group; row r of the batch has the table row ``table_rows[r]``, or r without it)."""
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
    _call("ms_decode_advance", prev_tokens.data_ptr(), token_ids.data_ptr(), positions.data_ptr(),
          context_lens.data_ptr(), n_live.data_ptr(), _ptr(table_rows), _ptr(draw_index), tp, sp, len(tables), width,
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


def _v_shape(k_pages: torch.Tensor, v_transposed: bool):
    P, nkv, page_size, d = k_pages.shape
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
    written.  K a multiple of 64 (else ``UnsupportedShape``)."""
    _check(a, "a", torch.bfloat16)
    _check(w, "w", torch.bfloat16, (None, a.shape[1]))
    if epilogue not in (EPI_STORE, EPI_SWIGLU):
        raise ValueError("the tiled product stores its result or the gated activation of it")
    M, K = a.shape
    N = w.shape[0]
    out = torch.empty((M, N // 2 if epilogue == EPI_SWIGLU else N), dtype=torch.bfloat16, device=a.device)
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
                            n_live_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n, h] = softmax(scale * q[n, h] . K[keys visible to n]) V, keys read in place from pages.

    q: [N, >= nh * d] (a row slice of the fused projection is fine), out [N, nh * d],
    pages [P, nkv, page_size, d] (values [P, nkv, d, page_size] with ``v_transposed``), block_table int32
    [rows, max_pages], token_req / positions int32 [N].
    Token n sees keys 0..positions[n] of request token_req[n] (the last ``window`` of them if given), whose
    pages are row ``table_rows[token_req[n]]`` of the table (row token_req[n] without ``table_rows``).  With
    ``n_live_tokens`` (a device int) tokens from that index on are left alone."""
    _check(k_pages, "k_pages")
    P, nkv, page_size, d = k_pages.shape
    _check(v_pages, "v_pages", k_pages.dtype, _v_shape(k_pages, v_transposed))
    _check(q, "q", k_pages.dtype, contiguous=False)
    N = q.shape[0]
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < num_heads * d:
        raise ValueError(f"q must be [N, >= {num_heads * d}] with unit stride along rows, got {list(q.shape)}")
    _check(out, "out", k_pages.dtype, (N, num_heads * d))
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
    _call("ms_paged_attention_generic", q.data_ptr(), q.stride(0) if N > 1 else q.shape[1], k_pages.data_ptr(),
          v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], _ptr(table_rows), _ptr(n_live_tokens),
          token_req.data_ptr(), positions.data_ptr(),
          out.data_ptr(), num_heads * d, N, num_heads, nkv, d, page_size, P, float(scale), int(window or 0),
          int(v_transposed), _code(q.dtype), _stream())
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
                         table_rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Matrix-core attention, bfloat16.  k_pages [P, nkv, page_size, d], vt_pages [P, nkv, d, page_size];
    request r owns tokens q_start[r]..q_start[r+1]-1, holds context_lens[r] keys after this step and has row
    ``table_rows[r]`` of ``block_table`` (row r without ``table_rows``).  ``max_q_len`` and ``max_context_len``
    are upper bounds; tokens from q_start[R] on belong to no request, a request may have no token.  A small
    batch of single tokens with long contexts also splits the keys over blocks (and combines)."""
    _check(k_pages, "k_pages", torch.bfloat16)
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
              int(window or 0), MIN_BLOCKS_PER_SPLIT, n_splits, _stream())
    else:
        _call("ms_paged_attention_mfma", q.data_ptr(), q_stride, k_pages.data_ptr(), vt_pages.data_ptr(),
              block_table.data_ptr(), block_table.shape[1], _ptr(table_rows), q_start.data_ptr(), context_lens.data_ptr(),
              out.data_ptr(), num_heads * d, R, N, max_q_len, num_heads, nkv, d, page_size, float(scale), int(window or 0),
              _stream())
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
                    window: Optional[int] = None) -> torch.Tensor:
    """Attention of a step's tokens (``ctx``: its StepContext) over a run's pages (``kv``: its KVView).
    bfloat16 with transposed value pages and a head size the matrix-core kernel has goes there; everything
    else (float32, other head sizes, small pages) goes to the generic kernel."""
    d, page_size = kv.k_pages.shape[3], kv.k_pages.shape[2]
    if q.dtype == torch.bfloat16 and not (kv.v_transposed and attention_mfma_supported(d, page_size)):
        _say_once(("attention", d, page_size),
                  f"bfloat16 attention with head size {d} and pages of {page_size} tokens runs on the vector-ALU kernel: "
                  f"the matrix-core kernel takes head sizes 32, 64 and 128 with pages of a multiple of 16")
    if (q.dtype == torch.bfloat16 and kv.v_transposed and attention_mfma_supported(d, page_size)
            and q.data_ptr() % 16 == 0 and (q.shape[0] == 1 or q.stride(0) % 8 == 0)):
        return paged_attention_mfma(q, kv.k_pages, kv.v_pages, kv.block_table, ctx.q_start, ctx.context_lens, out,
                                    num_heads, scale, ctx.max_q_len, ctx.max_context_len, window, kv.table_rows)
    return paged_attention_generic(q, kv.k_pages, kv.v_pages, kv.block_table, ctx.token_req, ctx.positions, out,
                                   num_heads, scale, window, kv.v_transposed, kv.table_rows, ctx.n_live_tokens)
