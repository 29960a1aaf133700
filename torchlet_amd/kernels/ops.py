"""Python face of the HIP kernels: one function per kernel entry point.

Every function takes ``torch`` tensors that already live on the GPU, checks shapes and
dtypes on the host (a kernel is never launched on operands it was not written for),
and launches on the current HIP stream.  Outputs are written into tensors the caller
allocated; nothing here allocates device memory except :func:`paged_attention`'s
split-merge scratch.  There is no CPU implementation: a missing library, or a tensor
that is not on the GPU, raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_void_p

import torch

from . import build as _build


class KernelError(RuntimeError):
    pass


_libs: dict[str, ctypes.CDLL] = {}

_DT = {torch.float32: 0, torch.bfloat16: 1}


def _lib(name: str) -> ctypes.CDLL:
    lib = _libs.get(name)
    if lib is None:
        try:
            path = _build.build(name)
        except _build.BuildError as exc:
            raise KernelError(f"kernel library {name!r} is not built and cannot be built here: {exc}") from exc
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as exc:
            raise KernelError(f"cannot load {path}: {exc}") from exc
        lib.tl_last_error.restype = ctypes.c_char_p
        _libs[name] = lib
        if name == "gemm" and torch.cuda.is_available():
            lib.tl_gemm_set_compute_units(c_int(compute_units()))
    return lib


def load(names) -> None:
    """Build (in parallel, if needed) and load the named libraries ahead of use."""
    missing = [n for n in names if n not in _libs]
    stale = [n for n in missing if not _build.is_current(n)]
    if stale:
        _build.build_many(stale)
    for n in missing:
        _lib(n)


MEASURED_COMPUTE_UNITS = 256      # the MI355X on which the kernels' plans were fitted
_compute_units: int | None = None


def compute_units() -> int:
    """The compute units of the current GPU, read from the device once; the matrix-product library's planners are
    told the same number, and parts that deal work to the compute units (how many parts a request's keys are cut
    into) get it from here.  Without a GPU: the MI355X's 256, for which the plans were measured."""
    global _compute_units
    if _compute_units is None:
        if not torch.cuda.is_available():
            return MEASURED_COMPUTE_UNITS
        _compute_units = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
        if "gemm" in _libs:
            _libs["gemm"].tl_gemm_set_compute_units(c_int(_compute_units))
    return _compute_units


def loaded_libraries() -> list[str]:
    return sorted(str(_build.lib_path(n)) for n in _libs)


def _check(lib: ctypes.CDLL, code: int) -> None:
    if code != 0:
        raise KernelError(lib.tl_last_error().decode())


def _ptr(t: torch.Tensor | None) -> c_void_p:
    if t is None:
        return c_void_p(0)
    if not t.is_cuda:
        raise KernelError(f"kernel operand on {t.device}; the kernels run on the GPU only")
    return c_void_p(t.data_ptr())


def _stream() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _dt(t: torch.Tensor, what: str) -> int:
    code = _DT.get(t.dtype)
    if code is None:
        raise KernelError(f"{what}: dtype {t.dtype} is not built (float32 and bfloat16 are)")
    return code


def _vec(t: torch.Tensor | None, n: int, what: str) -> int:
    """Check a weight/bias vector; returns 1 when it is float32, 0 for bfloat16."""
    if t is None:
        return 0
    if t.shape != (n,) or not t.is_contiguous():
        raise KernelError(f"{what}: expected a contiguous vector of {n}, got {tuple(t.shape)}")
    return 1 if _dt(t, what) == 0 else 0


def _i32(t: torch.Tensor | None, what: str, n: int | None = None) -> None:
    if t is None:
        return
    if t.dtype != torch.int32 or not t.is_contiguous() or (n is not None and t.numel() < n):
        raise KernelError(f"{what}: expected contiguous int32 of at least {n} elements, got {t.dtype} {tuple(t.shape)}")


# ----------------------------------------------------------------------------- ops

def embedding(token_ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """``out[t] = float(table[token_ids[t]]) * scale``; ``out`` is the 32-bit residual ``[T, H]``."""
    T = token_ids.numel()
    V, H = table.shape
    _i32(token_ids, "embedding ids", T)
    if out.shape != (T, H) or out.dtype != torch.float32 or not out.is_contiguous() or not table.is_contiguous():
        raise KernelError(f"embedding: out must be contiguous float32 [{T}, {H}], got {out.dtype} {tuple(out.shape)}")
    lib = _lib("elementwise")
    _check(lib, lib.tl_embedding(_ptr(token_ids), _ptr(table), c_int(_dt(table, "embedding table")), _ptr(out),
                                 c_int(T), c_int(H), c_int(V), c_float(scale), _stream()))


def add_rmsnorm(residual: torch.Tensor, pending: torch.Tensor | None, weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: torch.Tensor | None = None, gain: float = 1.0) -> None:
    """``r = residual (+ pending)``; ``out = r * (rsqrt(mean(r^2) + eps) * gain) * weight``.

    ``pending`` is ``[T, H]`` of the activation dtype, or float32 ``[P, T, H]``: slabs of partial
    sums (from :func:`linear_partials`) that are added up here.  Without ``rows`` every row is
    processed and ``r`` is written back into ``residual``; with ``rows`` (int32 source rows) only
    those are read and ``residual`` is untouched."""
    T, H = residual.shape
    n = T if rows is None else rows.numel()
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("add_rmsnorm: the residual must be contiguous float32")
    parts = 0
    if pending is not None:
        if pending.dim() == 3:
            parts = pending.shape[0]
            if pending.dtype != torch.float32 or pending.shape[1:] != residual.shape or not pending.is_contiguous():
                raise KernelError(f"add_rmsnorm: partial sums {pending.dtype} {tuple(pending.shape)} are not float32 [P, {T}, {H}]")
        elif pending.shape != residual.shape or pending.dtype != out.dtype or not pending.is_contiguous():
            raise KernelError(f"add_rmsnorm: pending {pending.dtype} {tuple(pending.shape)} does not match residual/out")
    if out.shape != (n, H) or not out.is_contiguous():
        raise KernelError(f"add_rmsnorm: out must be contiguous [{n}, {H}], got {tuple(out.shape)}")
    _i32(rows, "add_rmsnorm rows")
    wf = _vec(weight, H, "add_rmsnorm weight")
    lib = _lib("elementwise")
    _check(lib, lib.tl_add_rmsnorm(_ptr(residual), _ptr(pending), c_int(parts), c_int(T), _ptr(weight), c_int(wf),
                                   c_float(eps), c_float(gain), _ptr(out), _ptr(rows), c_int(n), c_int(H),
                                   c_int(_dt(out, "add_rmsnorm")), _stream()))


def linear_partials_pay(M: int, N: int, K: int) -> bool:
    """Whether a bfloat16 product whose consumer can add slabs up should come from
    :func:`linear_partials` (K a multiple of 64): up to 64 rows when its 64 x 64 output tiles are
    too few to fill the GPU (from 2 rows on; one row against a matrix of more than 4096 rows); with more rows
    when the library's estimate finds a tile shape with K split 2-8 ways faster than the best
    whole product, slabs included."""
    return bool(_lib("gemm").tl_gemm_partials_pay(c_int(M), c_int(N), c_int(K)))


def linear_partials(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``x @ weight.T`` as float32 slabs ``[P, M, N]`` of partial sums over P ranges of K (bfloat16
    operands, K a multiple of 8; more than 64 rows need a multiple of 64): for a product with too
    few output tiles to fill the GPU, where splitting K over work-groups does.  The slabs are
    summed by :func:`add_rmsnorm` (or by :func:`rope_cache_write`); P may be 1."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or weight.shape[1] != K or not weight.is_contiguous() or x.stride(1) != 1:
        raise KernelError("linear_partials: bfloat16 operands and fitting shapes only")
    lib = _lib("gemm")
    out = torch.empty((lib.tl_gemm_partials_parts(c_int(M), c_int(N), c_int(K)), M, N), dtype=torch.float32, device=x.device)
    parts = c_int(0)
    _check(lib, lib.tl_gemm_partials(_ptr(x), _ptr(weight), _ptr(out), c_int(M), c_int(N), c_int(K), c_int(x.stride(0)),
                                     ctypes.byref(parts), _stream()))
    return out[: parts.value]


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor,
           general: bool = False) -> None:
    """``out = x @ weight.T (+ bias)``; ``x [M, K]`` (rows may be strided), ``weight [N, K]``
    contiguous and of ``x``'s dtype, ``out [M, N]`` of that dtype or float32.  The library picks
    the kernel for the shape; ``general=True`` forces the general 32-bit-arithmetic kernel."""
    M, K = x.shape
    N, K2 = weight.shape
    if K2 != K or out.shape != (M, N):
        raise KernelError(f"linear: shapes x{tuple(x.shape)} w{tuple(weight.shape)} out{tuple(out.shape)} do not fit")
    if x.dtype != weight.dtype or x.stride(1) != 1 or out.stride(1) != 1 or not weight.is_contiguous():
        raise KernelError("linear: x and weight must share a dtype, weight contiguous, unit stride on the last axis")
    if out.dtype not in (x.dtype, torch.float32):
        raise KernelError(f"linear: out dtype {out.dtype} must be {x.dtype} or float32")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    entry = lib.tl_gemm_general if general else lib.tl_gemm
    _check(lib, entry(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N), c_int(K),
                                    c_int(x.stride(0)), c_int(out.stride(0)), c_int(_dt(x, "linear")),
                                    c_int(1 if out.dtype == torch.float32 else 0), _stream()))


def linear_f32_variant(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor, matrix_cores) -> None:
    """One named kernel of the 32-bit products (for tests and tuning): 0 / False the general tile kernel (``v_fma_f32``),
    1 / True the matrix-core tile kernel (``v_mfma_f32_32x32x2_f32``, K a multiple of 4), 2 and 3 the kernels for up to 16
    rows on multiply-adds and on the matrix cores (``v_mfma_f32_16x16x4_f32``); all multiply and add in true 32-bit."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.float32 or weight.dtype != torch.float32 or out.dtype != torch.float32 or out.shape != (M, N) \
            or weight.shape[1] != K or not weight.is_contiguous() or x.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("linear_f32_variant: float32 operands and fitting shapes only")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_f32_variant(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N), c_int(K),
                                        c_int(x.stride(0)), c_int(out.stride(0)), c_int(int(matrix_cores)), _stream()))


def linear_few_rows_variant(x, weight, bias, out, strips_per_wave: int, waves_along_k: int, rows_per_strip: int = 0) -> None:
    """One named instance of the few-rows matrix-core kernel (for tests and tuning); ``rows_per_strip``: the weight
    rows a work-group takes, up to 16 ``strips_per_wave`` (0: exactly that many)."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or out.shape != (M, N) or not weight.is_contiguous():
        raise KernelError("linear_few_rows_variant: bfloat16 operands and fitting shapes only")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_skinny_variant(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N),
                                           c_int(K), c_int(x.stride(0)), c_int(out.stride(0)),
                                           c_int(1 if out.dtype == torch.float32 else 0), c_int(strips_per_wave),
                                           c_int(waves_along_k), c_int(rows_per_strip), _stream()))


def linear_many_rows_variant(x, weight, bias, out, tile_m: int, tile_n: int, slab: int = 32) -> None:
    """One named tile shape of the many-rows matrix-core kernel (for tests and tuning)."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or out.shape != (M, N) or not weight.is_contiguous():
        raise KernelError("linear_many_rows_variant: bfloat16 operands and fitting shapes only")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_tile_variant(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N),
                                         c_int(K), c_int(x.stride(0)), c_int(out.stride(0)),
                                         c_int(1 if out.dtype == torch.float32 else 0), c_int(tile_m), c_int(tile_n), c_int(slab), _stream()))


DIRECT_TILES = ((64, 64), (64, 128), (64, 192), (64, 256), (64, 320), (128, 128), (128, 192), (128, 256), (256, 128), (192, 256), (256, 192), (256, 256), (256, 160))


def linear_direct_variant(x, weight, bias, out, tile_m: int, tile_n: int) -> None:
    """One named tile shape of the many-rows kernel that fetches its operands straight into
    shared memory (K a multiple of 64; for tests and tuning)."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or out.shape != (M, N) or not weight.is_contiguous():
        raise KernelError("linear_direct_variant: bfloat16 operands and fitting shapes only")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_direct_variant(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N),
                                           c_int(K), c_int(x.stride(0)), c_int(out.stride(0)),
                                           c_int(1 if out.dtype == torch.float32 else 0), c_int(tile_m), c_int(tile_n), _stream()))


def linear_direct_split_variant(x, weight, tile_m: int, tile_n: int, parts: int, stages: int = 0) -> torch.Tensor:
    """One named tile shape of the direct-load kernel with K split into ``parts``: float32 slabs
    ``[parts, M, N]`` (K a multiple of 64; ``stages=4`` with 128 x 128: the four-slab instance; for
    tests and tuning)."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or weight.shape[1] != K or not weight.is_contiguous() or x.stride(1) != 1:
        raise KernelError("linear_direct_split_variant: bfloat16 operands and fitting shapes only")
    out = torch.empty((parts, M, N), dtype=torch.float32, device=x.device)
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_direct_split_variant(_ptr(x), _ptr(weight), _ptr(out), c_int(M), c_int(N), c_int(K), c_int(x.stride(0)),
                                                 c_int(tile_m), c_int(tile_n), c_int(parts), c_int(stages), _stream()))
    return out


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The layout :func:`linear_swiglu` wants: blocks of 64 rows, 32 rows of ``gate`` then the
    32 rows of ``up`` with the same indices; the last block is padded with zero rows."""
    I, K = gate.shape
    blocks = -(-I // 32)
    g = torch.zeros((blocks * 32, K), dtype=gate.dtype, device=gate.device)
    u = torch.zeros_like(g)
    g[:I] = gate
    u[:I] = up
    return torch.stack((g.view(blocks, 32, K), u.view(blocks, 32, K)), dim=1).reshape(blocks * 64, K).contiguous()


def linear_swiglu(x: torch.Tensor, gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """``out = silu(x @ gate.T) * (x @ up.T)`` on the matrix cores with the gate applied to the
    32-bit accumulators; ``gate_up`` from :func:`interleave_gate_up`, bfloat16 only,
    ``x [M, K]`` with K a multiple of 8."""
    M, K = x.shape
    I = out.shape[1]
    if x.dtype != torch.bfloat16 or gate_up.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("linear_swiglu: bfloat16 only")
    if gate_up.shape != (-(-I // 32) * 64, K) or out.shape[0] != M or not gate_up.is_contiguous() or x.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError(f"linear_swiglu: shapes x{tuple(x.shape)} w{tuple(gate_up.shape)} out{tuple(out.shape)} do not fit")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_swiglu(_ptr(x), _ptr(gate_up), _ptr(out), c_int(M), c_int(I), c_int(K),
                                   c_int(x.stride(0)), c_int(out.stride(0)), _stream()))


def linear_swiglu_direct_variant(x: torch.Tensor, gate_up: torch.Tensor, out: torch.Tensor, tile_m: int, tile_n: int) -> None:
    """:func:`linear_swiglu` on one named tile shape of the kernel that fetches its operands straight into shared
    memory (K a multiple of 64; for tests and tuning)."""
    M, K = x.shape
    I = out.shape[1]
    if x.dtype != torch.bfloat16 or gate_up.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 \
            or gate_up.shape != (-(-I // 32) * 64, K) or out.shape[0] != M or not gate_up.is_contiguous() or x.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("linear_swiglu_direct_variant: bfloat16 operands and fitting shapes only")
    lib = _lib("gemm")
    _check(lib, lib.tl_gemm_swiglu_direct_variant(_ptr(x), _ptr(gate_up), _ptr(out), c_int(M), c_int(I), c_int(K),
                                                  c_int(x.stride(0)), c_int(out.stride(0)), c_int(tile_m), c_int(tile_n), _stream()))


def rope_cache_write(qkv: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int, rot_heads: int,
                     positions: torch.Tensor, inv_freq: torch.Tensor | None,
                     token_req: torch.Tensor | None = None, block_table: torch.Tensor | None = None,
                     k_plane: torch.Tensor | None = None, v_plane: torch.Tensor | None = None,
                     page_size: int = 0, pairs: bool = False, parts: torch.Tensor | None = None,
                     bias: torch.Tensor | None = None) -> None:
    """Rotate the first ``rot_heads`` heads of each row of ``qkv [T, >= (q+2kv)*hd]`` in
    place by the token's position (``inv_freq`` float32 ``[hd/2]``; ``None``: no rotation;
    ``pairs``: frequency j turns the neighbours ``(2j, 2j+1)`` instead of ``(j, j+hd/2)``)
    and, when planes are given, store rotated k and raw v of every token in its page:
    ``k_plane [pages, kv_heads, page, hd]``, ``v_plane [pages, kv_heads, hd, page]`` (values
    lie transposed inside a page).  With ``parts`` (float32 ``[P, T, width]``, slabs of partial
    sums of the projection, and its ``bias``) the rows are the sums of the slabs instead of what
    ``qkv`` holds: the queries are written to ``qkv``, keys and values to their pages only."""
    T = qkv.shape[0]
    if qkv.stride(1) != 1:
        raise KernelError("rope_cache_write: qkv needs unit stride on the last axis")
    _i32(positions, "positions", T)
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2):
        raise KernelError("rope_cache_write: inv_freq must be float32 [head_dim/2]")
    bt_stride = 0
    if k_plane is not None:
        _i32(token_req, "token_req", T)
        _i32(block_table, "block_table")
        bt_stride = block_table.stride(0)
        _check_planes("rope_cache_write", k_plane, v_plane, qkv.dtype, kv_heads, page_size, head_dim)
    num_parts = part_stride = parts_ld = bf = 0
    if parts is not None:
        if parts.dtype != torch.float32 or parts.dim() != 3 or parts.shape[1] != T or not parts.is_contiguous():
            raise KernelError("rope_cache_write: parts must be contiguous float32 [P, T, width]")
        num_parts, part_stride, parts_ld = parts.shape[0], parts.stride(0), parts.shape[2]
        bf = _vec(bias, parts_ld, "projection bias")
    elif bias is not None:
        raise KernelError("rope_cache_write: a bias comes with slabs of partial sums only")
    lib = _lib("elementwise")
    _check(lib, lib.tl_rope_cache_write(_ptr(qkv), c_int(qkv.stride(0)), c_int(T), c_int(q_heads), c_int(kv_heads),
                                        c_int(head_dim), c_int(rot_heads), _ptr(positions), _ptr(inv_freq), _ptr(token_req),
                                        _ptr(block_table), c_int(bt_stride), _ptr(k_plane), _ptr(v_plane), c_int(page_size),
                                        c_int(1 if pairs else 0), c_int(_dt(qkv, "rope_cache_write")),
                                        _ptr(parts), c_int(num_parts), ctypes.c_size_t(part_stride), c_int(parts_ld),
                                        _ptr(bias), c_int(bf), _stream()))


def pair_layout_rows(num_heads: int, head_dim: int) -> torch.Tensor:
    """Row order that turns a projection into the pair layout: within every head the rows
    ``j`` and ``j + head_dim/2`` (the two that frequency ``j`` of the split-half rotary encoding
    turns) become the neighbours ``2j`` and ``2j + 1``.  Scores are sums over the head's
    dimensions, so they do not change when queries and keys are reordered alike."""
    half = head_dim // 2
    within = torch.stack((torch.arange(half), torch.arange(half) + half), dim=1).reshape(-1)
    return (torch.arange(num_heads)[:, None] * head_dim + within[None, :]).reshape(-1)


def linear_rope_cache_write(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor,
                            q_heads: int, kv_heads: int, head_dim: int, positions: torch.Tensor, inv_freq: torch.Tensor,
                            token_req: torch.Tensor | None = None, block_table: torch.Tensor | None = None,
                            k_plane: torch.Tensor | None = None, v_plane: torch.Tensor | None = None,
                            page_size: int = 0) -> bool:
    """The query/key/value projection of a decode step with the rotation and the cache write in
    its epilogue: ``out[:, :q_heads*hd]`` gets the rotated queries; with planes given, ``weight``
    has ``(q_heads + 2 kv_heads) * hd`` rows and rotated keys and values go to their pages.  The
    rows of the query and key heads are in the pair layout (:func:`pair_layout_rows`).  Built
    for bfloat16 and up to 16 rows; returns ``False`` without doing anything for other shapes."""
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or M > 16 or M == 0 or head_dim % 4:
        return False
    if x.stride(1) != 1 or out.stride(1) != 1 or not weight.is_contiguous() or weight.shape[1] != K or out.shape[0] != M:
        raise KernelError("linear_rope_cache_write: shapes or strides do not fit")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2:
        raise KernelError("linear_rope_cache_write: inv_freq must be float32 [head_dim/2]")
    _i32(positions, "positions", M)
    bt_stride = 0
    if k_plane is not None:
        _i32(token_req, "token_req", M)
        _i32(block_table, "block_table")
        bt_stride = block_table.stride(0)
        _check_planes("linear_rope_cache_write", k_plane, v_plane, x.dtype, kv_heads, page_size, head_dim)
    if N != (q_heads + (2 * kv_heads if k_plane is not None else 0)) * head_dim or out.shape[1] < q_heads * head_dim:
        raise KernelError("linear_rope_cache_write: the projection's rows do not match the heads")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    rc = lib.tl_gemm_rope(_ptr(x), _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(M), c_int(N), c_int(K),
                          c_int(x.stride(0)), c_int(out.stride(0)), _ptr(positions), _ptr(inv_freq), _ptr(token_req),
                          _ptr(block_table), c_int(bt_stride), _ptr(k_plane), _ptr(v_plane), c_int(page_size),
                          c_int(q_heads), c_int(kv_heads), c_int(head_dim), _stream())
    if rc == 100:          # not built for this shape
        return False
    _check(lib, rc)
    return True


def _norm_args(what: str, residual: torch.Tensor, pending: torch.Tensor | None, weight: torch.Tensor, eps: float,
               residual_out: torch.Tensor):
    """The arguments that describe ``norm(residual + pending)`` of one row to a kernel that makes it itself."""
    H = residual.shape[-1]
    if residual.dtype != torch.float32 or residual_out.dtype != torch.float32 or residual.numel() != H or residual_out.numel() != H \
            or not residual.is_contiguous() or not residual_out.is_contiguous():
        raise KernelError(f"{what}: the residual and its successor must be one contiguous float32 row")
    parts = part_stride = 0
    if pending is not None:
        if pending.dim() == 3:
            if pending.dtype != torch.float32 or pending.shape[1:] != (1, H) or not pending.is_contiguous():
                raise KernelError(f"{what}: partial sums {pending.dtype} {tuple(pending.shape)} are not float32 [P, 1, {H}]")
            parts, part_stride = pending.shape[0], pending.stride(0)
        elif pending.dtype != torch.bfloat16 or pending.numel() != H or not pending.is_contiguous():
            raise KernelError(f"{what}: pending {pending.dtype} {tuple(pending.shape)} is not a bfloat16 row of {H}")
    wf = _vec(weight, H, f"{what} norm weight")
    return (_ptr(residual), _ptr(residual_out), _ptr(pending), c_int(parts), ctypes.c_long(part_stride), _ptr(weight), c_int(wf),
            c_float(eps))


def linear_rope_cache_write_normed(residual: torch.Tensor, pending: torch.Tensor | None, norm_weight: torch.Tensor, eps: float,
                                   residual_out: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None,
                                   out: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int, positions: torch.Tensor,
                                   inv_freq: torch.Tensor, token_req: torch.Tensor | None = None,
                                   block_table: torch.Tensor | None = None, k_plane: torch.Tensor | None = None,
                                   v_plane: torch.Tensor | None = None, page_size: int = 0) -> bool:
    """:func:`linear_rope_cache_write` for ONE row whose input is ``norm(residual + pending)`` (see
    :func:`add_rmsnorm`), made inside the kernel: ``residual [1, K]`` float32, ``pending`` bfloat16
    ``[1, K]``, float32 slabs ``[P, 1, K]`` or ``None``; the sum goes to ``residual_out`` (another
    tensor than ``residual``).  Returns ``False`` without doing anything for shapes it is not built for."""
    K = residual.shape[-1]
    N = weight.shape[0]
    if weight.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or residual.shape[0] != 1 or head_dim % 4:
        return False
    if out.stride(1) != 1 or not weight.is_contiguous() or weight.shape[1] != K or out.shape[0] != 1:
        raise KernelError("linear_rope_cache_write_normed: shapes or strides do not fit")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2:
        raise KernelError("linear_rope_cache_write_normed: inv_freq must be float32 [head_dim/2]")
    _i32(positions, "positions", 1)
    bt_stride = 0
    if k_plane is not None:
        _i32(token_req, "token_req", 1)
        _i32(block_table, "block_table")
        bt_stride = block_table.stride(0)
        _check_planes("linear_rope_cache_write_normed", k_plane, v_plane, torch.bfloat16, kv_heads, page_size, head_dim)
    if N != (q_heads + (2 * kv_heads if k_plane is not None else 0)) * head_dim or out.shape[1] < q_heads * head_dim:
        raise KernelError("linear_rope_cache_write_normed: the projection's rows do not match the heads")
    bf = _vec(bias, N, "linear bias")
    lib = _lib("gemm")
    rc = lib.tl_gemm_rope_normed(*_norm_args("linear_rope_cache_write_normed", residual, pending, norm_weight, eps, residual_out),
                                 _ptr(weight), _ptr(bias), c_int(bf), _ptr(out), c_int(N), c_int(K), c_int(out.stride(0)),
                                 _ptr(positions), _ptr(inv_freq), _ptr(token_req), _ptr(block_table), c_int(bt_stride),
                                 _ptr(k_plane), _ptr(v_plane), c_int(page_size), c_int(q_heads), c_int(kv_heads),
                                 c_int(head_dim), _stream())
    if rc == 100:          # not built for this shape
        return False
    _check(lib, rc)
    return True


def linear_swiglu_normed(residual: torch.Tensor, pending: torch.Tensor | None, norm_weight: torch.Tensor, eps: float,
                         residual_out: torch.Tensor, gate_up: torch.Tensor, out: torch.Tensor) -> bool:
    """:func:`linear_swiglu` for ONE row whose input is ``norm(residual + pending)``, made inside the
    kernel (see :func:`linear_rope_cache_write_normed`).  Returns ``False`` without doing anything
    for shapes it is not built for."""
    K = residual.shape[-1]
    I = out.shape[1]
    if gate_up.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or residual.shape[0] != 1:
        return False
    if gate_up.shape != (-(-I // 32) * 64, K) or out.shape[0] != 1 or not gate_up.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"linear_swiglu_normed: shapes w{tuple(gate_up.shape)} out{tuple(out.shape)} do not fit a row of {K}")
    lib = _lib("gemm")
    rc = lib.tl_gemm_swiglu_normed(*_norm_args("linear_swiglu_normed", residual, pending, norm_weight, eps, residual_out),
                                   _ptr(gate_up), _ptr(out), c_int(I), c_int(K), _stream())
    if rc == 100:
        return False
    _check(lib, rc)
    return True


def _check_planes(what, k_plane, v_plane, dtype, kv_heads, page_size, head_dim) -> None:
    for p, shape in ((k_plane, (kv_heads, page_size, head_dim)), (v_plane, (kv_heads, head_dim, page_size))):
        if p.dtype != dtype or p.dim() != 4 or tuple(p.shape[1:]) != shape or not p.is_contiguous():
            raise KernelError(f"{what}: plane {tuple(p.shape)} {p.dtype} is not [pages, {', '.join(map(str, shape))}] {dtype}")
    if k_plane.shape[0] != v_plane.shape[0]:
        raise KernelError(f"{what}: key and value planes differ in their number of pages")


ATTENTION_ROWS = 16   # rows (tokens x heads of one group) a work-group owns


def attention_library(head_dim: int) -> str:
    """The attention library that serves ``head_dim``: one is compiled per multiple of 16 and takes the seven even
    sizes below it too (its general kernel pads them inside; the matrix-core kernels are for the multiple itself)."""
    if head_dim % 2 or not 2 <= head_dim <= 256:
        raise KernelError(f"attention kernels take even head sizes from 2 to 256, not {head_dim}")
    return f"attention_hd{-(-head_dim // 16) * 16}"

SPLIT_SCRATCH_BYTES = 256 << 20     # most memory the parts of a split attention may take before they are merged


def attention_tile_tokens(num_heads: int, num_kv_heads: int) -> int:
    """New tokens of one request that share a tile, given the group size."""
    group = num_heads // num_kv_heads
    return max(1, ATTENTION_ROWS // min(group, ATTENTION_ROWS))


def paged_attention(q: torch.Tensor, out: torch.Tensor, k_plane: torch.Tensor, v_plane: torch.Tensor,
                    block_table: torch.Tensor, req_indptr: torch.Tensor, ctx_lens: torch.Tensor,
                    tile_req: torch.Tensor, tile_tok0: torch.Tensor, num_tiles: int, tile_tokens: int,
                    num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, window: int,
                    scale: float, splits: int = 1, general: bool = False, merge_tokens=None, waves: int = 4) -> None:
    """Causal attention of the step's tokens over their requests' cached keys.

    ``q [T, >= heads*hd]`` (row-strided view), ``out [T, heads*hd]``, ``k_plane [pages,
    kv_heads, page, hd]``, ``v_plane [pages, kv_heads, hd, page]``, ``block_table [R,
    max_blocks]`` int32; the new token ``i`` of request ``r`` sits at position
    ``ctx_lens[r] + i``.  ``window`` 0: all keys.  bfloat16 with pages of a multiple of 4
    tokens runs on the matrix cores; ``general=True`` forces the general kernel.  When the
    tiles cover only some of the step's tokens and ``splits > 1``, ``merge_tokens = (int32
    indices of those tokens, their number)`` keeps the merge of the parts to their rows.
    ``tile_req = tile_tok0 = None``: every request brings exactly one token, token ``i`` that of
    request ``i`` (a decode step); the kernel then looks nothing up before it asks for the
    request's length, block table and query.  ``waves``: 4 or 8 to a work-group of the matrix-core kernel
    (they deal a part's keys among themselves; the other kernels take no notice)."""
    T = q.shape[0]
    if waves not in (4, 8):
        raise KernelError("paged_attention: work-groups of 4 or 8 waves")
    if q.stride(1) != 1 or out.shape != (T, num_heads * head_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("paged_attention: q/out shapes or dtypes do not fit")
    _check_planes("paged_attention", k_plane, v_plane, q.dtype, num_kv_heads, page_size, head_dim)
    for name, t in (("block_table", block_table), ("ctx_lens", ctx_lens)):
        _i32(t, name)
    if tile_req is None:        # every request brings one token: tile i is the token of request i
        if tile_tok0 is not None or num_tiles != T or ctx_lens.numel() < T or block_table.shape[0] < T:
            raise KernelError("paged_attention: without a tile list every request brings exactly one token")
        req_indptr = None
    else:
        for name, t in (("req_indptr", req_indptr), ("tile_req", tile_req), ("tile_tok0", tile_tok0)):
            _i32(t, name)
        if tile_req.numel() < num_tiles or tile_tok0.numel() < num_tiles:
            raise KernelError("paged_attention: tile arrays shorter than the number of tiles")
    if merge_tokens is not None:
        _i32(merge_tokens[0], "merge_tokens", merge_tokens[1])
    part_o = part_ml = None
    # the parts are indexed by the step's tokens: a few decode tokens beside a long portion would make the
    # scratch large for nothing, so the split count gives way (fewer parts: the same result up to rounding)
    padded = -(-head_dim // 16) * 16            # the parts are as wide as the library's head size
    splits = max(1, min(splits, SPLIT_SCRATCH_BYTES // (T * num_heads * (padded + 2) * 4)))
    if splits > 1:
        part_o = torch.empty((T * num_heads * splits, padded), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * num_heads * splits, 2), dtype=torch.float32, device=q.device)
    lib = _lib(attention_library(head_dim))
    _check(lib, lib.tl_paged_attention(_ptr(q), c_int(q.stride(0)), _ptr(out), _ptr(k_plane), _ptr(v_plane),
                                       _ptr(block_table), c_int(block_table.stride(0)), _ptr(req_indptr), _ptr(ctx_lens),
                                       _ptr(tile_req), _ptr(tile_tok0), c_int(num_tiles), c_int(T), c_int(tile_tokens),
                                       c_int(num_heads), c_int(num_kv_heads), c_int(head_dim), c_int(page_size), c_int(window),
                                       c_float(scale), c_int(splits), _ptr(part_o), _ptr(part_ml),
                                       _ptr(merge_tokens[0]) if merge_tokens is not None else c_void_p(None),
                                       c_int(merge_tokens[1] if merge_tokens is not None else 0),
                                       c_int(_dt(q, "paged_attention")), c_int(1 if general else 0), c_int(waves), _stream()))


PREFILL_ATTENTION_ROWS = 64      # rows a work-group of the prompt-portion kernel owns
PREFILL_ATTENTION_MAX_HEAD_DIM = 128


def prefill_attention_tile_tokens(num_heads: int, num_kv_heads: int) -> int:
    group = num_heads // num_kv_heads
    return max(1, PREFILL_ATTENTION_ROWS // min(group, ATTENTION_ROWS))


def paged_attention_prefill(q: torch.Tensor, out: torch.Tensor, k_plane: torch.Tensor, v_plane: torch.Tensor,
                            block_table: torch.Tensor, req_indptr: torch.Tensor, ctx_lens: torch.Tensor,
                            tile_req: torch.Tensor, tile_tok0: torch.Tensor, num_tiles: int, tile_tokens: int,
                            num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, window: int,
                            scale: float) -> None:
    """The attention of :func:`paged_attention` for prompt portions: bfloat16, head sizes up
    to 128, pages of a multiple of 4 tokens; tiles of ``tile_tokens`` tokens (64 rows) whose keys
    and values pass through shared memory once per work-group.  Writes the rows of its tiles only."""
    T = q.shape[0]
    if q.dtype != torch.bfloat16 or head_dim > PREFILL_ATTENTION_MAX_HEAD_DIM or head_dim % 16 or page_size % 4:
        raise KernelError("paged_attention_prefill: bfloat16, head sizes that are multiples of 16 up to 128 and pages of a multiple of 4 tokens only")
    if q.stride(1) != 1 or out.shape != (T, num_heads * head_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("paged_attention_prefill: q/out shapes or dtypes do not fit")
    _check_planes("paged_attention_prefill", k_plane, v_plane, q.dtype, num_kv_heads, page_size, head_dim)
    for name, t in (("block_table", block_table), ("req_indptr", req_indptr), ("ctx_lens", ctx_lens),
                    ("tile_req", tile_req), ("tile_tok0", tile_tok0)):
        _i32(t, name)
    if tile_req.numel() < num_tiles or tile_tok0.numel() < num_tiles:
        raise KernelError("paged_attention_prefill: tile arrays shorter than the number of tiles")
    lib = _lib(f"attention_hd{head_dim}")
    _check(lib, lib.tl_paged_attention_prefill(_ptr(q), c_int(q.stride(0)), _ptr(out), _ptr(k_plane), _ptr(v_plane),
                                               _ptr(block_table), c_int(block_table.stride(0)), _ptr(req_indptr),
                                               _ptr(ctx_lens), _ptr(tile_req), _ptr(tile_tok0), c_int(num_tiles),
                                               c_int(tile_tokens), c_int(num_heads), c_int(num_kv_heads), c_int(page_size),
                                               c_int(window), c_float(scale), _stream()))


PROMPT_ATTENTION_ROWS = 128      # rows a work-group of the 128-row prompt kernel owns
PROMPT_ATTENTION_HEAD_DIMS = (64, 128)


PROMPT_ATTENTION_MAX_BLOCKS = 2048     # pages of a sequence whose block-table entries a work-group keeps in shared memory


def prompt_attention_fits(dtype: torch.dtype, head_dim: int, page_size: int, max_blocks: int = 0, scale: float = 1.0) -> bool:
    """Whether :func:`paged_attention_prompt` is built for this case: bfloat16, head size 64 or
    128, pages of 8, 16, 32, ... tokens, sequences of up to 2048 pages (``max_blocks``: the
    longest sequence of the step in pages), a positive factor on the scores."""
    return (dtype == torch.bfloat16 and head_dim in PROMPT_ATTENTION_HEAD_DIMS and page_size >= 8
            and page_size & (page_size - 1) == 0 and max_blocks <= PROMPT_ATTENTION_MAX_BLOCKS and scale > 0)


def prompt_attention_tile_tokens(num_heads: int, num_kv_heads: int) -> int:
    group = num_heads // num_kv_heads
    return max(1, PROMPT_ATTENTION_ROWS // min(group, PROMPT_ATTENTION_ROWS))


def paged_attention_prompt(q: torch.Tensor, out: torch.Tensor, k_plane: torch.Tensor, v_plane: torch.Tensor,
                           block_table: torch.Tensor, req_indptr: torch.Tensor, ctx_lens: torch.Tensor,
                           tile_req: torch.Tensor, tile_tok0: torch.Tensor, num_tiles: int, tile_tokens: int,
                           num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, window: int,
                           scale: float, max_total_len: int | None = None, splits: int = 1,
                           merge_tokens: tuple[torch.Tensor, int] | None = None) -> None:
    """The attention of :func:`paged_attention` for prompt portions in tiles of 128 rows
    (``tile_tokens`` tokens times the heads of a group): bfloat16, head size 64 or 128, pages
    of a multiple of 8 tokens; keys and values go straight into shared memory once per
    work-group.  Writes the rows of its tiles only.  ``max_total_len``: the longest sequence of the
    step (cached + new tokens; default: what the block table could hold).  ``splits`` > 1 deals
    every tile's keys to that many work-groups (for few tiles against long sequences) and merges
    their parts for the tokens listed in ``merge_tokens`` (int32 indices, how many): the tokens
    of the tiles' requests."""
    T = q.shape[0]
    used_blocks = block_table.shape[1] if max_total_len is None else min(block_table.shape[1], -(-max_total_len // page_size))
    if not prompt_attention_fits(q.dtype, head_dim, page_size, used_blocks):
        raise KernelError("paged_attention_prompt: bfloat16, head size 64 or 128, pages of 8, 16, 32, ... tokens and "
                          f"sequences of up to {PROMPT_ATTENTION_MAX_BLOCKS} pages only")
    if q.stride(1) != 1 or out.shape != (T, num_heads * head_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("paged_attention_prompt: q/out shapes or dtypes do not fit")
    _check_planes("paged_attention_prompt", k_plane, v_plane, q.dtype, num_kv_heads, page_size, head_dim)
    for name, t in (("block_table", block_table), ("req_indptr", req_indptr), ("ctx_lens", ctx_lens),
                    ("tile_req", tile_req), ("tile_tok0", tile_tok0)):
        _i32(t, name)
    if tile_req.numel() < num_tiles or tile_tok0.numel() < num_tiles:
        raise KernelError("paged_attention_prompt: tile arrays shorter than the number of tiles")
    lib = _lib(f"attention_hd{head_dim}")
    part_o = part_ml = tokens = None
    count = 0
    if splits > 1:
        if merge_tokens is None or merge_tokens[1] <= 0:
            raise KernelError("paged_attention_prompt: splits > 1 need the tokens whose parts are merged")
        tokens, count = merge_tokens
        _i32(tokens, "merge_tokens")
        if tokens.numel() < count:
            raise KernelError("paged_attention_prompt: merge_tokens shorter than its count")
        splits = max(1, min(splits, SPLIT_SCRATCH_BYTES // (T * num_heads * (head_dim + 2) * 4)))
        part_o = torch.empty((T * num_heads * splits, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T * num_heads * splits, 2), dtype=torch.float32, device=q.device)
    _check(lib, lib.tl_paged_attention_prompt(_ptr(q), c_int(q.stride(0)), _ptr(out), _ptr(k_plane), _ptr(v_plane),
                                              _ptr(block_table), c_int(block_table.stride(0)), _ptr(req_indptr),
                                              _ptr(ctx_lens), _ptr(tile_req), _ptr(tile_tok0), c_int(num_tiles),
                                              c_int(tile_tokens), c_int(num_heads), c_int(num_kv_heads), c_int(page_size),
                                              c_int(window), c_float(scale), c_int(max(1, used_blocks)),
                                              c_int(splits), _ptr(part_o), _ptr(part_ml), _ptr(tokens), c_int(count), _stream()))


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """``out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i]``."""
    T, I2 = gate_up.shape
    if I2 % 2 or out.shape != (T, I2 // 2) or out.dtype != gate_up.dtype or not out.is_contiguous() or not gate_up.is_contiguous():
        raise KernelError("swiglu: shapes or dtypes do not fit")
    lib = _lib("elementwise")
    _check(lib, lib.tl_swiglu(_ptr(gate_up), _ptr(out), c_int(T), c_int(I2 // 2), c_int(_dt(out, "swiglu")), _stream()))


def sample(logits: torch.Tensor, temperature: torch.Tensor | None, keys: torch.Tensor | None, out: torch.Tensor) -> None:
    """Token per row of float32 ``logits [N, V]``: arg max where ``temperature`` is 0 (or
    absent), else a Gumbel-max draw from ``softmax(logits / temperature)`` seeded by the
    row's int32 ``keys`` entry."""
    N, V = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be float32 with unit stride on the last axis")
    if temperature is not None and (temperature.dtype != torch.float32 or temperature.numel() < N or not temperature.is_contiguous()):
        raise KernelError("sample: temperature must be contiguous float32 [N]")
    _i32(keys, "sample keys", N)
    _i32(out, "sample out", N)
    lib = _lib("sampling")
    scratch = torch.empty((2, N, lib.tl_sample_chunks(c_int(V))), dtype=torch.int32, device=logits.device)
    _check(lib, lib.tl_sample(_ptr(logits), c_int(N), c_int(V), c_int(logits.stride(0)), _ptr(temperature), _ptr(keys),
                              _ptr(out), _ptr(scratch), _stream()))


def stream_read(data: torch.Tensor, groups: int = 0) -> torch.Tensor:
    """Read every byte of ``data`` (contiguous, on the GPU) once with a kernel that does nothing else, and
    return the exclusive-or of its 32-bit words per work-group (int32; ``groups`` work-groups, 0: the default).  A yardstick: the time it takes is
    what this GPU needs to deliver that much memory to a kernel, whatever the kernel does with it."""
    if not data.is_contiguous() or data.data_ptr() % 16 or data.numel() * data.element_size() < 16:
        raise KernelError("stream_read: contiguous, 16-byte aligned memory of at least 16 bytes")
    lib = _lib("elementwise")
    lib.tl_stream_read.argtypes = [c_void_p, ctypes.c_size_t, c_void_p, c_int, c_void_p]
    sink = torch.empty(groups or lib.tl_stream_read_groups(), dtype=torch.int32, device=data.device)
    _check(lib, lib.tl_stream_read(_ptr(data), ctypes.c_size_t(data.numel() * data.element_size()), _ptr(sink), c_int(groups), _stream()))
    return sink
