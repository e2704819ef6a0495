"""Python face of the HIP kernels: shape / dtype / device checks, then one C call.

Every function works on tensors that live on the GPU and launches on torch's current
stream.  There is no CPU path: a tensor on the CPU, or a kernel library that cannot
be built or loaded, is an error.

Dispatch rule: bfloat16 operands whose sizes the matrix-core kernels take go to those
kernels (module "bf16"); everything else - float32, mixed storage types, odd sizes -
goes to the general kernels (module "core"), which take any size.
``use_fast_kernels(False)`` forces the general kernels (tests compare the two).
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..errors import KernelError
from . import _lib
from .workspace import KernelWorkspace, KeyRanges, Partials, stream_layout, stream_layout_takes

PI_F32, PI_BF16 = 0, 1
MAX_HEAD_DIM = 256              # the matrix-core attention kernels
GENERAL_MAX_HEAD_DIM = 640      # the general attention kernel (key rows of a latent cache are wide)

_FAST = True


def use_fast_kernels(enabled: bool) -> bool:
    """Switch the matrix-core kernels on or off; returns the previous setting."""
    global _FAST
    prev, _FAST = _FAST, bool(enabled)
    return prev


def fast_kernels_enabled() -> bool:
    return _FAST


def ensure_loaded(dtype: torch.dtype) -> None:
    """Build / load what a model of compute dtype ``dtype`` needs."""
    _lib.load("core")
    if dtype == torch.bfloat16 and _FAST and _lib.build.MODULES["bf16"]:
        _lib.load("bf16")


# ----------------------------------------------------------------------------- helpers
def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return PI_F32
    if t.dtype == torch.bfloat16:
        return PI_BF16
    raise KernelError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}")


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernels run on the GPU only; got a tensor on " + str(t.device))


def _stream() -> int:
    return _lib.current_stream()


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride (elements) of a 2-D tensor whose rows are dense."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{what}: expected a 2-D tensor with dense rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t: torch.Tensor, what: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what}: expected a contiguous int32 tensor, got {t.dtype}")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what}: expected at least {n} entries, got {t.numel()}")


def check_attention_sizes(num_heads: int, num_kv_heads: int, head_dim: int) -> None:
    """Sizes the attention kernels take; anything else is refused here, by name."""
    if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
        raise KernelError(f"attention: {num_heads} heads is not a positive multiple of {num_kv_heads} kv heads")
    if head_dim <= 0 or head_dim % 16 or head_dim > MAX_HEAD_DIM:
        raise KernelError(f"attention: head_dim {head_dim} must be a multiple of 16 up to {MAX_HEAD_DIM}")


def check_general_attention_sizes(num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int) -> None:
    """Sizes the general attention kernel takes (the only one for heads with options)."""
    if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
        raise KernelError(f"attention: {num_heads} heads is not a positive multiple of {num_kv_heads} kv heads")
    if not (0 < head_dim <= GENERAL_MAX_HEAD_DIM and 0 < value_dim <= GENERAL_MAX_HEAD_DIM):
        raise KernelError(f"attention: head sizes {head_dim} / {value_dim} must be at most {GENERAL_MAX_HEAD_DIM}")


# ----------------------------------------------------------------------------- ops
def embedding(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0,
              pos_table: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None) -> None:
    """out[t, :] = float32(table[ids[t], :]) * scale; with a learned position table,
    out[t, :] = table[ids[t], :] * scale + pos_table[positions[t], :]."""
    _gpu(out, table, ids, pos_table, positions)
    T, D = out.shape
    if out.dtype != torch.float32 or not out.is_contiguous():
        raise KernelError("embedding: output must be contiguous float32")
    if table.dim() != 2 or table.shape[1] != D or not table.is_contiguous():
        raise KernelError(f"embedding: table shape {tuple(table.shape)} does not match width {D}")
    _i32(ids, "embedding ids", T)
    if pos_table is not None:
        if pos_table.dim() != 2 or pos_table.shape[1] != D or not pos_table.is_contiguous() or pos_table.dtype != table.dtype:
            raise KernelError(f"embedding: position table {tuple(pos_table.shape)} {pos_table.dtype} does not match [*, {D}] {table.dtype}")
        _i32(positions, "embedding positions", T)
        _lib.call("core", "pi_embedding_positions", out.data_ptr(), table.data_ptr(), pos_table.data_ptr(), _dt(table), ids.data_ptr(),
                  positions.data_ptr(), float(scale), T, D, table.shape[0], pos_table.shape[0], _stream())
        return
    _lib.call("core", "pi_embedding", out.data_ptr(), table.data_ptr(), _dt(table), ids.data_ptr(), T, D,
              table.shape[0], float(scale), _stream())


def softcap_(x: torch.Tensor, cap: float) -> None:
    """x <- cap * tanh(x / cap), in place, float32."""
    _gpu(x)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("softcap: expected a contiguous float32 tensor")
    if not cap > 0.0:
        raise KernelError(f"softcap: the cap must be positive, got {cap}")
    _lib.call("core", "pi_softcap", x.data_ptr(), x.numel(), float(cap), _stream())


def rmsnorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float,
            rows: Optional[torch.Tensor] = None, ws: Optional[KernelWorkspace] = None) -> None:
    """out[m, :] = weight * x[r, :] / sqrt(mean(x[r, :]^2) + eps), r = rows[m] (or m).  An update of
    ``x`` that is still pending in ``ws`` is added first, in the same pass, and written back to
    ``x`` (with ``rows``: to those rows only; the others are not read again by this caller)."""
    _gpu(out, x, weight, rows)
    M, D = out.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or x.dim() != 2 or x.shape[1] != D:
        raise KernelError(f"rmsnorm: input must be contiguous float32 [*, {D}], got {x.dtype} {tuple(x.shape)}")
    if not out.is_contiguous() or weight.shape != (D,) or not weight.is_contiguous():
        raise KernelError(f"rmsnorm: output must be contiguous and weight [{D}], got weight {tuple(weight.shape)}")
    if rows is None:
        if x.shape[0] != M:
            raise KernelError(f"rmsnorm: {x.shape[0]} input rows for {M} output rows")
    else:
        _i32(rows, "rmsnorm rows", M)
    pending = ws.take_pending(x) if ws is not None else None
    if pending is not None:
        ws.counts["added_by_norm"] += 1
    part, splits = (pending.part.data_ptr(), pending.splits) if pending is not None else (None, 0)
    _lib.call("core", "pi_rmsnorm", out.data_ptr(), _dt(out), x.data_ptr(), _ptr(rows), weight.data_ptr(),
              _dt(weight), float(eps), M, D, part, splits, x.shape[0], _stream())


# ----------------------------------------------------------------------------- deferred updates
# A product into the residual stream whose k-range was split over blocks may stay in pieces
# (``Partials`` in the caller's ``KernelWorkspace``) until the next reader of the stream:
# ``rmsnorm`` folds the sum of the pieces and the residual add into its own pass.  Whoever reads
# the stream in any other way calls ``materialize`` first.  Only callers that pass
# ``may_defer=True`` and a workspace to ``gemm`` ever leave an update pending (one at most per
# workspace), and a block arrangement must materialize before it hands the stream to a part that
# does not read it through ``rmsnorm``.
def materialize(x: torch.Tensor, ws: Optional[KernelWorkspace]) -> torch.Tensor:
    """Apply an update of ``x`` that is still pending in ``ws``, if there is one."""
    p = ws.take_pending(x) if ws is not None else None
    if p is not None:
        from . import fast
        fast.reduce_into(x, p, accumulate=True)
        ws.counts["applied"] += 1
    return x


def reset_deferred(ws: Optional[KernelWorkspace]) -> None:
    """Forget a pending update (start of a step: nothing of an earlier, failed step may linger)."""
    if ws is not None:
        ws.pending = None


def discard_deferred(x: torch.Tensor, ws: Optional[KernelWorkspace]) -> None:
    """Forget a pending update of ``x`` (the stream is not read again)."""
    if ws is not None and ws.take_pending(x) is not None:
        ws.counts["discarded"] += 1


def swiglu(out: torch.Tensor, gate_up: torch.Tensor, block: int = 0) -> None:
    """out[t, i] = silu(gate) * up.  ``block`` = 0: gate in columns [0, I), up in [I, 2I);
    ``block`` = b: gate and up interleaved in blocks of b columns."""
    _gpu(out, gate_up)
    T, I = out.shape
    if gate_up.shape != (T, 2 * I) or gate_up.dtype != out.dtype or not (out.is_contiguous() and gate_up.is_contiguous()):
        raise KernelError(f"swiglu: expected gate_up [{T}, {2 * I}] of {out.dtype}, got {tuple(gate_up.shape)} {gate_up.dtype}")
    if block < 0 or (block and I % block):
        raise KernelError(f"swiglu: interleave block {block} does not divide {I}")
    _lib.call("core", "pi_swiglu", out.data_ptr(), gate_up.data_ptr(), _dt(out), T, I, int(block), _stream())


def gemm_swiglu(out: torch.Tensor, a: torch.Tensor, w_gate_up: torch.Tensor, block: int = 0,
                ws: Optional[KernelWorkspace] = None) -> None:
    """out[M, I] = silu(a @ Wg^T) * (a @ Wu^T) where ``w_gate_up`` [2I, K] holds the gate and
    up rows in halves (``block`` 0) or interleaved in blocks of ``block`` rows.  With bfloat16
    operands and blocks of 16 the product and the activation are one kernel."""
    _gpu(out, a, w_gate_up)
    M, I = out.shape
    if w_gate_up.shape[0] != 2 * I or a.shape != (M, w_gate_up.shape[1]) or out.dtype != a.dtype:
        raise KernelError(f"gemm_swiglu: shapes do not agree: a {tuple(a.shape)}, w {tuple(w_gate_up.shape)}, out {tuple(out.shape)}")
    if M == 0:
        return
    if _FAST and block == 16 and a.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and out.is_contiguous():
        from . import fast
        if fast.gemm_swiglu(out, a, w_gate_up, M, 2 * I, a.shape[1], _rows(a, "gemm a"), _rows(w_gate_up, "gemm w"), ws):
            return
    gu = torch.empty((M, 2 * I), dtype=a.dtype, device=a.device)
    gemm(gu, a, w_gate_up, ws=ws)
    swiglu(out, gu, block)


def gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, accumulate: bool = False,
         may_defer: bool = False, ws: Optional[KernelWorkspace] = None) -> None:
    """out[M, N] (+)= a[M, K] @ w[N, K]^T with float32 accumulation.

    ``ws``: where a product split over k keeps its pieces (without one, memory of this call's own).
    ``may_defer`` (with ``accumulate`` and ``ws``): the caller promises that ``out`` is next read
    by ``rmsnorm`` or ``materialize`` with the same workspace; a product that was split over k may
    then stay in pieces there."""
    if isinstance(a, KeyRanges):
        # attention's output of a decode step, its key ranges not merged yet: the weight-streaming
        # kernel merges them as it reads; anything else gets them merged first
        _gpu(out, w)
        if w.dim() != 2 or out.shape != (a.tokens, w.shape[0]) or w.shape[1] != a.heads * a.head_dim:
            raise KernelError(f"gemm: shapes do not agree: ranges [{a.tokens}, {a.heads} x {a.head_dim}], w {tuple(w.shape)}, out {tuple(out.shape)}")
        if accumulate:
            if out.dtype != torch.float32:
                raise KernelError("gemm: accumulation needs a float32 output")
            materialize(out, ws)
        from . import fast
        if _FAST and fast.gemm_from_ranges(out, a, w, accumulate, w.shape[0], _rows(w, "gemm w"), _rows(out, "gemm out"),
                                           may_defer and accumulate and out.is_contiguous(), ws):
            return
        merged = torch.empty((a.tokens, a.heads * a.head_dim), dtype=torch.bfloat16, device=out.device)
        fast.merge_ranges(merged, a)
        a = merged
    _gpu(out, a, w)
    if a.dim() != 2 or w.dim() != 2 or out.dim() != 2:
        raise KernelError("gemm: operands must be 2-D")
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or out.shape != (M, N):
        raise KernelError(f"gemm: shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    if accumulate and out.dtype != torch.float32:
        raise KernelError("gemm: accumulation needs a float32 output")
    lda, ldw, ldc = _rows(a, "gemm a"), _rows(w, "gemm w"), _rows(out, "gemm out")
    if M == 0:
        return
    if accumulate:
        materialize(out, ws)
    if _FAST and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        from . import fast
        if fast.gemm(out, a, w, accumulate, M, N, K, lda, ldw, ldc, may_defer and accumulate and out.is_contiguous(), ws):
            return
    _lib.call("core", "pi_gemm_general", out.data_ptr(), _dt(out), ldc, a.data_ptr(), _dt(a), lda, w.data_ptr(),
              _dt(w), ldw, M, N, K, int(accumulate), _stream())


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, hd: int, page_size: int, dtype, vd: Optional[int] = None) -> int:
    """Keys [pages, kv_heads, page, head_dim]; values transposed, [pages, kv_heads, value width (= head_dim unless given), page]."""
    vd = hd if vd is None else vd
    if (k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (nkv, page_size, hd)
            or tuple(v_cache.shape) != (k_cache.shape[0], nkv, vd, page_size)):
        raise KernelError(f"cache: expected keys [pages, {nkv}, {page_size}, {hd}] and values [pages, {nkv}, {vd}, {page_size}], "
                          f"got {tuple(k_cache.shape)} / {tuple(v_cache.shape)}")
    if k_cache.dtype != dtype or v_cache.dtype != dtype or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise KernelError(f"cache: must be contiguous {dtype}, got {k_cache.dtype}")
    return k_cache.shape[0]


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, magnitude: float = 1.0) -> torch.Tensor:
    """float32 [T, 2 * half]: cos then sin of float32(position) * inv_freq[j], for every token, each
    times ``magnitude`` (a scaled rotation that also stretches the rotated pairs)."""
    _gpu(positions, inv_freq)
    T, half = positions.shape[0], inv_freq.numel()
    _i32(positions, "positions")
    if inv_freq.dtype != torch.float32 or not inv_freq.is_contiguous():
        raise KernelError("rope: the frequency table must be contiguous float32")
    table = torch.empty((T, 2 * half), dtype=torch.float32, device=positions.device)
    _lib.call("core", "pi_rope_table", table.data_ptr(), positions.data_ptr(), inv_freq.data_ptr(), T, half, float(magnitude), _stream())
    return table


def _rotary_args(rotary, positions, T):
    """(table pointer, rotary_dim, interleaved) from ``rotary`` = (frequencies or table, R, interleaved)."""
    if rotary is None:
        return None, 0, False, None
    src, rdim, inter = rotary
    if src.dim() == 2:                       # already the step's cos / sin table
        if src.shape != (T, rdim) or src.dtype != torch.float32 or not src.is_contiguous():
            raise KernelError(f"rope: cos / sin table must be contiguous float32 [{T}, {rdim}]")
        return src.data_ptr(), rdim, inter, src
    if src.numel() != rdim // 2:
        raise KernelError(f"rope: frequency table must be float32 [{rdim // 2}]")
    table = rope_table(positions, src)
    return table.data_ptr(), rdim, inter, table


def qkv_projection(h: torch.Tensor, w_qkv: torch.Tensor, dtype: torch.dtype, ws: Optional[KernelWorkspace] = None):
    """h @ w_qkv^T for the attention mixer: a tensor [T, N] in ``dtype``, or - when the
    product was split over k and there is a workspace to keep them in - its pieces
    (``Partials``), which ``rope_kv_write`` sums on the fly so that the rotation sees float32
    values.  The pieces are good until the next product with the same workspace."""
    if _FAST and ws is not None and h.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16 and h.is_cuda:
        from . import fast
        p = fast.gemm_pieces(h, w_qkv, ws)
        if p is not None:
            ws.counts["qkv_pieces"] += 1
            return p
    out = torch.empty((h.shape[0], w_qkv.shape[0]), dtype=dtype, device=h.device)
    gemm(out, h, w_qkv, ws=ws)
    return out


def rope_kv_write(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor], positions: torch.Tensor,
                  req_of_token: torch.Tensor, rotary, num_heads: int, num_kv_heads: int, head_dim: int,
                  k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  block_table: Optional[torch.Tensor], page_size: int, pieces=None, write_kv: Optional[bool] = None,
                  value_dim: Optional[int] = None, bias: Optional[torch.Tensor] = None) -> None:
    """Rotate q in place by each token's position; rotate k and store k, v into the pages.
    ``value_dim``: the width of a value head when it differs from ``head_dim``.

    ``rotary`` = (inv_freq float32 [R/2] or the step's cos / sin table [T, R], R, interleaved), or
    None for no rotation.
    ``k``/``v`` None: queries only (the layer reads a cache that another one writes).
    ``pieces``: the q|k|v projection still split over k (``fast.Partials`` with columns
    [q heads | k heads | v heads]); then ``q`` is the output buffer for the rotated queries and
    ``k``/``v`` are not given (``write_kv`` says whether the cache is written).
    ``bias``: float32, one per column of the projection [q heads | k heads | v heads]; it is added in float32 before
    the rotation (with ``pieces``: to their sum, so the biased projection is never held in reduced precision).
    """
    _gpu(q, k, v, positions, req_of_token, k_cache, v_cache, block_table, bias)
    T = q.shape[0]
    vd = head_dim if value_dim is None else int(value_dim)
    if bias is not None:
        with_kv = bool(write_kv) if pieces is not None else k is not None
        need = num_heads * head_dim + (num_kv_heads * (head_dim + vd) if with_kv else 0)
        if bias.dtype != torch.float32 or not bias.is_contiguous() or bias.numel() < need:
            raise KernelError(f"rope: the projection's bias must be contiguous float32 with at least {need} entries")
    if value_dim is None:
        check_attention_sizes(num_heads, num_kv_heads, head_dim)
    else:
        check_general_attention_sizes(num_heads, num_kv_heads, head_dim, vd)
    if q.shape[1] != num_heads * head_dim:
        raise KernelError(f"rope: q has {q.shape[1]} columns, expected {num_heads * head_dim}")
    _i32(positions, "positions", T)
    if pieces is not None:
        write = bool(write_kv)
        table_ptr, rdim, inter, _keep = _rotary_args(rotary, positions, T)
        q_size, kv_size = num_heads * head_dim, num_kv_heads * head_dim
        if pieces.M != T or pieces.N < q_size + (kv_size + num_kv_heads * vd if write else 0):
            raise KernelError(f"rope: pieces [{pieces.M}, {pieces.N}] do not hold q, k, v of {T} tokens")
        pages = _check_cache(k_cache, v_cache, num_kv_heads, head_dim, page_size, q.dtype, vd) if write else 0
        _lib.call(
            "core", "pi_rope_kv_write", q.data_ptr(), _rows(q, "q"), None, 0, None, 0, _dt(q), positions.data_ptr(),
            _ptr(req_of_token) if write else None, table_ptr, rdim, int(bool(inter)), T, num_heads, num_kv_heads,
            head_dim, int(write), _ptr(k_cache) if write else None, _ptr(v_cache) if write else None,
            _ptr(block_table) if write else None, block_table.shape[1] if write else 0, page_size if write else 0, pages,
            pieces.part.data_ptr(), pieces.splits, pieces.N, 0, q_size, q_size + kv_size, vd, _ptr(bias), _stream())
        return
    write = k is not None
    table_ptr, rdim, inter, _keep = _rotary_args(rotary, positions, T)
    if not write and rdim == 0 and bias is None:
        return
    pages = 0
    if write:
        if (v is None or k.shape != (T, num_kv_heads * head_dim) or v.shape != (T, num_kv_heads * vd) or k.dtype != q.dtype
                or v.dtype != q.dtype):
            raise KernelError(f"rope: k / v must be [{T}, {num_kv_heads * head_dim}] / [{T}, {num_kv_heads * vd}] of {q.dtype}")
        pages = _check_cache(k_cache, v_cache, num_kv_heads, head_dim, page_size, q.dtype, vd)
        _i32(req_of_token, "req_of_token", T)
        if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
            raise KernelError("rope: block table must be contiguous int32 [requests, width]")
    _lib.call(
        "core", "pi_rope_kv_write", q.data_ptr(), _rows(q, "q"), _ptr(k), _rows(k, "k") if write else 0, _ptr(v),
        _rows(v, "v") if write else 0, _dt(q), positions.data_ptr(), _ptr(req_of_token) if write else None,
        table_ptr, rdim, int(bool(inter)), T, num_heads, num_kv_heads, head_dim, int(write),
        _ptr(k_cache) if write else None, _ptr(v_cache) if write else None, _ptr(block_table) if write else None,
        block_table.shape[1] if write else 0, page_size if write else 0, pages, None, 0, 0, 0,
        num_heads * head_dim, num_heads * head_dim + num_kv_heads * head_dim, vd, _ptr(bias), _stream())


def decode_attention_from_projection(out: torch.Tensor, qkv, ctx, rotary, num_heads: int, num_kv_heads: int,
                                     head_dim: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                                     block_table: torch.Tensor, page_size: int, scale: float, window: int,
                                     write_kv: bool, ws: Optional[KernelWorkspace] = None, leave_ranges: int = 0):
    """For a step that holds single tokens only: rotation, cache write and attention in one
    kernel, from the q|k|v projection ``qkv`` (a tensor [T, N] or ``fast.Partials``, columns
    [q heads | k heads | v heads]).  Returns False, having done nothing, when the step, the
    sizes or the rotation (``rotary`` as for ``rope_kv_write``; only the whole head with paired
    halves, or none) are not what that kernel serves; the caller then takes the separate kernels.
    ``leave_ranges`` (needs ``ws``; 0, or the bytes of the weight matrix the result goes to): the
    caller hands the result straight to ``gemm`` with that matrix; when the keys were split into
    ranges, the kernel may then return them unmerged (``KeyRanges``, in the workspace) instead of
    filling ``out``, and the product merges them as it reads."""
    if not (_FAST and out.dtype == torch.bfloat16 and out.is_cuda and getattr(ctx, "all_decode", False)):
        return False
    from . import fast
    if not isinstance(qkv, Partials) and qkv.dtype != torch.bfloat16:
        return False
    T = out.shape[0]
    table = None
    if rotary is not None:
        src, rdim, inter = rotary
        if rdim != head_dim or inter:
            return False
        _ptr_unused, _rdim, _inter, table = _rotary_args(rotary, ctx.positions, T)
    check_attention_sizes(num_heads, num_kv_heads, head_dim)
    if out.shape != (T, num_heads * head_dim):
        raise KernelError(f"attention: out {tuple(out.shape)} does not match {num_heads} x {head_dim}")
    pages = _check_cache(k_cache, v_cache, num_kv_heads, head_dim, page_size, out.dtype)
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
        raise KernelError("attention: block table must be contiguous int32 [requests, width]")
    return fast.decode_attention_from_projection(out, qkv, ctx, table, num_heads, num_kv_heads, head_dim, k_cache, v_cache,
                                                 block_table, page_size, scale, window, pages, write_kv, ws, leave_ranges)


def _f32_vector(t: Optional[torch.Tensor], n: int, what: str) -> None:
    if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n or not t.is_cuda):
        raise KernelError(f"{what}: expected contiguous float32 with {n} entries on the GPU, got {t.dtype} {tuple(t.shape)}")


def paged_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, ctx, num_heads: int, num_kv_heads: int, head_dim: int,
                    page_size: int, scale: float, window: int = 0, ws: Optional[KernelWorkspace] = None, *,
                    value_dim: Optional[int] = None, slopes: Optional[torch.Tensor] = None,
                    sinks: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                    softcap: float = 0.0, out_scale: float = 1.0, chunk: int = 0) -> None:
    """Causal attention of every token of the step over its request's pages.

    ``ctx`` carries ``positions`` and ``req_of_token`` ([T] int32), the step's shape on the host
    (``q_lens``, ``kv_lens``, ``all_decode``) and, in ``plans``, the work lists that the
    matrix-core kernels want (made here when the step function has not).

    Options: ``value_dim`` (values of another width than keys; ``out`` is then [T, heads * value_dim]),
    ``slopes`` (float32 [heads]: slope * distance is taken off a key's scaled score), ``sinks``
    (float32 [heads]: exp(sink) joins the softmax's denominator once), ``gate`` (float32
    [T, heads]: multiplies a head's output), ``softcap`` (c > 0: the scaled score s becomes c * tanh(s / c)),
    ``out_scale`` (a factor on every output, applied in float32 before the one rounding), ``chunk`` (C > 0: positions
    are cut into chunks of C, counted from 0, and a token sees the keys of its own chunk only).
    """
    _gpu(out, q, k_cache, v_cache, block_table, ctx.positions, ctx.req_of_token)
    chunk = int(chunk or 0)
    if chunk < 0:
        raise KernelError(f"attention: a chunk must be positive, got {chunk}")
    T = q.shape[0]
    vd = head_dim if value_dim is None else int(value_dim)
    softcap, out_scale = float(softcap or 0.0), float(out_scale)
    if softcap < 0.0:
        raise KernelError(f"attention: a cap on the scores must be positive, got {softcap}")
    plain = value_dim is None and slopes is None and sinks is None and gate is None and softcap == 0.0 and out_scale == 1.0
    if plain:
        check_attention_sizes(num_heads, num_kv_heads, head_dim)
    else:
        check_general_attention_sizes(num_heads, num_kv_heads, head_dim, vd)
        _f32_vector(slopes, num_heads, "attention slopes")
        _f32_vector(sinks, num_heads, "attention sinks")
        _f32_vector(gate, T * num_heads, "attention gate")
    if q.shape[1] != num_heads * head_dim or out.shape != (T, num_heads * vd) or out.dtype != q.dtype:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not match {num_heads} x {head_dim} (values {vd})")
    pages = _check_cache(k_cache, v_cache, num_kv_heads, head_dim, page_size, q.dtype, vd)
    _i32(ctx.positions, "positions", T)
    _i32(ctx.req_of_token, "req_of_token", T)
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
        raise KernelError("attention: block table must be contiguous int32 [requests, width]")
    if T == 0:
        return
    if _FAST and q.dtype == torch.bfloat16 and vd == head_dim and head_dim % 16 == 0 and (plain or scale > 0):
        # the matrix-core kernels take heads whose values are as wide as their keys, options included
        from . import fast
        if fast.paged_attention(out, q, k_cache, v_cache, block_table, ctx, num_heads, num_kv_heads, head_dim,
                                page_size, scale, window, pages, ws, slopes, sinks, gate, softcap, out_scale, chunk):
            return
    # a step of few tokens over long contexts: its keys cut into ranges, merged by a second kernel
    # (as many as the context-length bucket asks for, so that a step gives the same bits eagerly and replayed)
    # (chunks bound a token's keys whatever the context: one range)
    ranges = general_attention_ranges(T, num_heads, min(int(ctx.max_kv_len), chunk) if chunk else int(ctx.max_kv_len))
    part = torch.empty(T * num_heads * ranges * (vd + 2), dtype=torch.float32, device=q.device) if ranges > 1 else None
    _lib.call("core", "pi_paged_attention_general", out.data_ptr(), _rows(out, "attention out"), q.data_ptr(),
              _rows(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(), _dt(q), block_table.data_ptr(),
              block_table.shape[1], ctx.req_of_token.data_ptr(), ctx.positions.data_ptr(), T, num_heads,
              num_kv_heads, head_dim, page_size, float(scale), int(window), pages, ranges, _ptr(part),
              0 if part is None else part.numel(), vd, _ptr(slopes), _ptr(sinks), _ptr(gate), softcap, out_scale, chunk, _stream())


def general_attention_ranges(tokens: int, num_heads: int, max_kv_len: int) -> int:
    """Key ranges per (token, head) that the general attention kernel makes for such a step."""
    return int(_lib.load("core").pi_paged_attention_general_ranges(tokens, num_heads, decode_length_bucket(max_kv_len)))


def sample(out: torch.Tensor, logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           uniform: Optional[torch.Tensor] = None, ws: Optional[KernelWorkspace] = None) -> None:
    """out[m] = argmax of row m (lowest index among equals) where temperature[m] <= 0 or
    no temperatures are given; otherwise the first index whose cumulative
    softmax(logits / temperature) reaches uniform[m]."""
    _gpu(out, logits, temperature, uniform)
    M, V = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("sample: logits must be float32")
    _i32(out, "sample out", M)
    for t, what in ((temperature, "temperature"), (uniform, "uniform")):
        if t is not None and (t.dtype != torch.float32 or t.numel() < M or not t.is_contiguous()):
            raise KernelError(f"sample: {what} must be contiguous float32 [{M}]")
    if temperature is not None and uniform is None:
        raise KernelError("sample: temperatures given without uniform numbers")
    chunks = _lib.load("core").pi_sample_chunks(V)
    if chunks == 0:
        part = None
    elif ws is not None:
        part = ws.sample_part
    else:
        part = torch.empty(M * chunks * 4, dtype=torch.float32, device=logits.device)
    _lib.call("core", "pi_sample", out.data_ptr(), logits.data_ptr(), _rows(logits, "logits"), _ptr(temperature),
              _ptr(uniform), M, V, _ptr(part), 0 if part is None else part.numel(), _stream())


# ----------------------------------------------------------------------------- work lists
def decode_length_bucket(max_kv_len: int) -> int:
    """The context-length bucket that decides a decode step's attention key ranges."""
    from . import fast
    return fast.decode_length_bucket(max_kv_len)


def attention_planner(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                      window: int, device, chunk: int = 0):
    """What makes a step's work lists for an attention mixer of these sizes (a hashable object with
    ``plan(q_lens, kv_lens)``; equal ones share a plan), or None when its kernels need none."""
    if _FAST and dtype == torch.bfloat16 and _lib.build.MODULES["bf16"]:
        from . import fast
        return fast.attention_planner(dtype, num_heads, num_kv_heads, head_dim, page_size, int(window), torch.device(device), int(chunk or 0))
    return None


def upload_arrays(arrays, device):
    """int32 host arrays by name -> device views of one packed copy."""
    from . import fast
    return fast.upload_arrays(arrays, device)


# ----------------------------------------------------------------------------- streams normalised on the way out
def cast_stream(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The float32 stream in the activation type (itself when that is float32)."""
    _gpu(x)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("cast: the stream must be contiguous float32")
    if dtype == torch.float32:
        return x
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    _lib.call("core", "pi_cast_stream", out.data_ptr(), _dt(out), x.data_ptr(), x.numel(), _stream())
    return out


def layer_norm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float,
               rows: Optional[torch.Tensor] = None) -> None:
    """out[m, :] = (x[r, :] - mean) / sqrt(mean of squared deviations + eps) * weight + bias, r = rows[m] (or m);
    ``x`` float32, weight and bias float32, everything computed in float32 and rounded once into ``out``."""
    _gpu(out, x, weight, bias, rows)
    M, D = out.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or x.dim() != 2 or x.shape[1] != D or not out.is_contiguous():
        raise KernelError(f"layer norm: input must be contiguous float32 [*, {D}], got {x.dtype} {tuple(x.shape)}")
    _f32_vector(weight, D, "layer norm weight")
    _f32_vector(bias, D, "layer norm bias")
    if rows is None:
        if x.shape[0] != M:
            raise KernelError(f"layer norm: {x.shape[0]} input rows for {M} output rows")
    else:
        _i32(rows, "layer norm rows", M)
    _lib.call("core", "pi_layer_norm", out.data_ptr(), _dt(out), x.data_ptr(), _ptr(rows), weight.data_ptr(), bias.data_ptr(),
              float(eps), M, D, x.shape[0], _stream())


def sandwich_norm_add(x: torch.Tensor, a: torch.Tensor, post, eps: float, nxt=None, h_dtype: Optional[torch.dtype] = None,
                      w_a: Optional[torch.Tensor] = None, b: Optional[torch.Tensor] = None, w_b: Optional[torch.Tensor] = None,
                      a_bias: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x += LN(y; post) with y = a (+ a_bias), or rms(a (+ a_bias); w_a), or the mean of rms(a (+ a_bias); w_a) and
    rms(b; w_b); LN the layer norm with (weight, bias) = ``post``, rms(v; w) = v / sqrt(mean(v^2) + eps) * w; all
    float32.  With ``nxt`` = (weight, bias) the layer norm of the new stream is returned in ``h_dtype`` (what the next
    sublayer reads), made in the same pass."""
    _gpu(x, a, b, w_a, w_b, a_bias)
    T, D = x.shape
    for t, what in ((x, "stream"), (a, "result"), (b, "second result")):
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != (T, D)):
            raise KernelError(f"norm and add: the {what} must be contiguous float32 [{T}, {D}]")
    vectors = [(post[0], "norm weight"), (post[1], "norm bias"), (w_a, "branch weight"), (w_b, "second branch weight"), (a_bias, "result bias")]
    if nxt is not None:
        vectors += [(nxt[0], "next norm weight"), (nxt[1], "next norm bias")]
    for t, what in vectors:
        _f32_vector(t, D, f"norm and add {what}")
    h = None
    if nxt is not None:
        h = torch.empty((T, D), dtype=h_dtype or torch.float32, device=x.device)
    _lib.call("core", "pi_sandwich_norm_add", x.data_ptr(), _ptr(h), _dt(h) if h is not None else PI_F32, a.data_ptr(), _ptr(a_bias),
              _ptr(w_a), _ptr(b), _ptr(w_b), post[0].data_ptr(), post[1].data_ptr(), _ptr(nxt[0]) if nxt is not None else None,
              _ptr(nxt[1]) if nxt is not None else None, float(eps), T, D, _stream())
    return h


def diff_combine(out: torch.Tensor, attn: torch.Tensor, lam: float, eps: float, mult: float, heads: int, kv_heads: int,
                 value_dim: int, split: int = 1) -> None:
    """Two attention maps per head into one result: ``attn`` [T, 2 * heads * value_dim] holds the maps as heads of
    their own, a head's values in ``split`` equal pieces that were attended as heads of their own, in the order
    [kv group][map][piece][head within the group]; out[t, n, :] = mult * o / sqrt(mean(o^2) + eps) with
    o = map 1 - lam * map 2 of head n, float32 arithmetic."""
    _gpu(out, attn)
    T = out.shape[0]
    if tuple(out.shape) != (T, heads * value_dim) or tuple(attn.shape) != (T, 2 * heads * value_dim) or not (out.is_contiguous() and attn.is_contiguous()):
        raise KernelError(f"two maps: expected contiguous [{T}, {2 * heads * value_dim}] -> [{T}, {heads * value_dim}], got {tuple(attn.shape)} -> {tuple(out.shape)}")
    _lib.call("core", "pi_diff_combine", out.data_ptr(), _dt(out), attn.data_ptr(), _dt(attn), float(lam), float(eps), float(mult), T,
              int(heads), int(kv_heads), int(value_dim), int(split), _stream())


EPI_RELU2 = 5        # the matrix-core products' epilogue: max(c, 0)^2 rounded to bfloat16


def gemm_relu_squared(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, ws: Optional[KernelWorkspace] = None) -> None:
    """out[M, N] = max(a @ w^T, 0)^2, the square taken on the product's float32 result.  With bfloat16 operands and more
    rows than the weight-streaming products take, product and activation are one kernel."""
    _gpu(out, a, w)
    M, N = out.shape
    if w.shape[0] != N or a.shape != (M, w.shape[1]):
        raise KernelError(f"gemm_relu_squared: shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    if M == 0:
        return
    if _FAST and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and out.is_contiguous():
        from . import fast
        if fast.gemm_relu_squared(out, a, w, M, N, a.shape[1], _rows(a, "gemm a"), _rows(w, "gemm w")):
            return
    u = torch.empty((M, N), dtype=torch.float32, device=a.device)
    gemm(u, a, w, ws=ws)
    relu_squared(out, u)


def relu_squared(out: torch.Tensor, a: torch.Tensor) -> None:
    """out = max(a, 0)^2 from float32 ``a`` into ``out`` (any type), squared before the one rounding."""
    _gpu(out, a)
    if a.dtype != torch.float32 or out.shape != a.shape or not (a.is_contiguous() and out.is_contiguous()):
        raise KernelError("squared relu: expected a contiguous float32 input and an output of its shape")
    _lib.call("core", "pi_relu_squared", out.data_ptr(), _dt(out), a.data_ptr(), a.numel(), _stream())


def branch_norm_add(x: torch.Tensor, a: torch.Tensor, w_outer: torch.Tensor, eps: float, mult: float,
                    w_a: Optional[torch.Tensor] = None, b: Optional[torch.Tensor] = None, w_b: Optional[torch.Tensor] = None,
                    h_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """x += mult * norm(y; w_outer) with y = a, or norm(a; w_a), or the mean of norm(a; w_a) and
    norm(b; w_b); norm(v; w) = v / sqrt(mean(v^2) + eps) * w, all float32.  With ``h_dtype`` the new
    stream is also returned in that type (the stream itself for float32)."""
    _gpu(x, a, b, w_outer, w_a, w_b)
    T, D = x.shape
    for t, what in ((x, "stream"), (a, "branch"), (b, "second branch")):
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != (T, D)):
            raise KernelError(f"branch norm: the {what} must be contiguous float32 [{T}, {D}]")
    for t, what in ((w_outer, "outer weight"), (w_a, "branch weight"), (w_b, "second branch weight")):
        _f32_vector(t, D, f"branch norm {what}")
    h = None
    if h_dtype is not None and h_dtype != torch.float32:
        h = torch.empty((T, D), dtype=h_dtype, device=x.device)
    _lib.call("core", "pi_branch_norm_add", x.data_ptr(), _ptr(h), _dt(h) if h is not None else PI_F32, a.data_ptr(), _ptr(w_a),
              _ptr(b), _ptr(w_b), w_outer.data_ptr(), float(eps), float(mult), T, D, _stream())
    if h_dtype is None:
        return None
    return x if h is None else h


def qk_norm_kv_write(q_out: torch.Tensor, gate_out: Optional[torch.Tensor], proj: torch.Tensor, w_q: Optional[torch.Tensor],
                     w_k: Optional[torch.Tensor], ctx, eps: float, temp_coef: float, temp_every: int, num_heads: int,
                     num_kv_heads: int, head_dim: int, value_dim: int, num_gates: int, k_cache: Optional[torch.Tensor],
                     v_cache: Optional[torch.Tensor], block_table: Optional[torch.Tensor], page_size: int,
                     per_head: bool = False, has_kv: bool = True) -> None:
    """From float32 projection rows [q | k | v | gates] (a tensor, or ``Partials``: the product still split over k,
    whose pieces are added here): queries and keys each normalised over their
    WHOLE row (all heads at once; weights float32, None: no norm), queries times the position's
    temperature 1 + coef * ln(floor((p + 1) / every) + 1), keys and values into their pages,
    gates through a sigmoid into ``gate_out`` (float32 [T, num_gates]).
    ``per_head``: every head of q and k is divided by the root mean square of its own entries instead (weights, when
    given, still multiply).  ``has_kv`` False: the rows hold [q | gates] only (keys and values are another layer's)."""
    pieces = proj if isinstance(proj, Partials) else None
    _gpu(q_out, gate_out, pieces.part if pieces is not None else proj, w_q, w_k, k_cache, v_cache, block_table)
    T = q_out.shape[0]
    QN = num_heads * head_dim
    KN, VN = (num_kv_heads * head_dim, num_kv_heads * value_dim) if has_kv else (0, 0)
    if not has_kv and k_cache is not None:
        raise KernelError("qk norm: a cache to write without keys and values in the projection")
    if pieces is not None:
        if pieces.M != T or pieces.N < QN + KN + VN + num_gates:
            raise KernelError(f"qk norm: pieces [{pieces.M}, {pieces.N}] do not hold q, k, v and gates of {T} tokens")
    elif proj.dtype != torch.float32 or proj.dim() != 2 or proj.shape[0] != T or proj.shape[1] < QN + KN + VN + num_gates:
        raise KernelError(f"qk norm: projection must be float32 [{T}, >= {QN + KN + VN + num_gates}], got {proj.dtype} {tuple(proj.shape)}")
    if q_out.shape[1] != QN:
        raise KernelError(f"qk norm: q has {q_out.shape[1]} columns, expected {QN}")
    _f32_vector(w_q, QN, "qk norm query weight")
    _f32_vector(w_k if has_kv else None, KN, "qk norm key weight")
    if num_gates and (gate_out is None or gate_out.dtype != torch.float32 or not gate_out.is_contiguous() or gate_out.numel() != T * num_gates):
        raise KernelError(f"qk norm: gates need contiguous float32 [{T}, {num_gates}]")
    pages = 0
    if k_cache is not None:
        pages = _check_cache(k_cache, v_cache, num_kv_heads, head_dim, page_size, q_out.dtype, value_dim)
        if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
            raise KernelError("qk norm: block table must be contiguous int32 [requests, width]")
    _i32(ctx.positions, "positions", T)
    _i32(ctx.req_of_token, "req_of_token", T)
    _lib.call("core", "pi_qk_norm_kv_write", q_out.data_ptr(), _rows(q_out, "q"), _ptr(gate_out), _dt(q_out),
              None if pieces is not None else proj.data_ptr(), pieces.N if pieces is not None else _rows(proj, "projection"),
              _ptr(w_q), _ptr(w_k), ctx.positions.data_ptr(), ctx.req_of_token.data_ptr(), float(eps),
              float(temp_coef), int(temp_every), T, num_heads, num_kv_heads, head_dim, value_dim, num_gates, _ptr(k_cache),
              _ptr(v_cache), _ptr(block_table), block_table.shape[1] if k_cache is not None else 0, page_size, pages,
              pieces.part.data_ptr() if pieces is not None else None, pieces.splits if pieces is not None else 0,
              pieces.M * pieces.N if pieces is not None else 0, int(bool(per_head)), int(bool(has_kv)), _stream())


# ----------------------------------------------------------------------------- attention through a latent
def latent_kv_write(cq_out: Optional[torch.Tensor], proj, w_q: Optional[torch.Tensor], w_kv: torch.Tensor, table: Optional[torch.Tensor],
                    ctx, eps: float, q_rank: int, kv_rank: int, rot: int, k_cache: Optional[torch.Tensor],
                    v_cache: Optional[torch.Tensor], block_table: Optional[torch.Tensor], page_size: int) -> None:
    """From float32 projection rows [query latent: q_rank | key/value latent: kv_rank | shared rotated key part: rot]
    (a tensor, or ``Partials``): the query latent RMS-normalised with ``w_q`` into ``cq_out`` ([T, q_rank], the
    activation type); the key/value latent RMS-normalised with ``w_kv`` and the rotated part turned by the token's
    angles (``table``: the step's [T, rot] cosines and sines, neighbouring pairs) into the pages: keys
    [pages, 1, page, kv_rank + rot] = [latent | rotated part], values transposed [pages, 1, kv_rank (+ rot), page]."""
    pieces = proj if isinstance(proj, Partials) else None
    _gpu(cq_out, pieces.part if pieces is not None else proj, w_q, w_kv, table, k_cache, v_cache, block_table)
    N = q_rank + kv_rank + rot
    if pieces is not None:
        T = pieces.M
        if pieces.N < N:
            raise KernelError(f"latent: pieces [{pieces.M}, {pieces.N}] do not hold {N} columns")
    else:
        T = proj.shape[0]
        if proj.dtype != torch.float32 or proj.dim() != 2 or proj.shape[1] < N:
            raise KernelError(f"latent: projection must be float32 [{T}, >= {N}], got {proj.dtype} {tuple(proj.shape)}")
    if q_rank and (cq_out is None or cq_out.shape != (T, q_rank)):
        raise KernelError(f"latent: the query latent's place must be [{T}, {q_rank}]")
    _f32_vector(w_q, q_rank, "latent query norm weight")
    _f32_vector(w_kv, kv_rank, "latent key norm weight")
    if rot and (table is None or table.shape != (T, rot) or table.dtype != torch.float32 or not table.is_contiguous()):
        raise KernelError(f"latent: cos / sin table must be contiguous float32 [{T}, {rot}]")
    pages, v_rows = 0, kv_rank
    dtype = cq_out.dtype if cq_out is not None else (k_cache.dtype if k_cache is not None else torch.float32)
    if k_cache is not None:
        v_rows = v_cache.shape[2] if v_cache.dim() == 4 else -1
        if v_rows not in (kv_rank, kv_rank + rot):
            raise KernelError(f"latent: values of {v_rows} rows are neither the latent's {kv_rank} nor the key's {kv_rank + rot}")
        pages = _check_cache(k_cache, v_cache, 1, kv_rank + rot, page_size, dtype, v_rows)
        if block_table.dim() != 2 or block_table.dtype != torch.int32 or not block_table.is_contiguous():
            raise KernelError("latent: block table must be contiguous int32 [requests, width]")
    _i32(ctx.positions, "positions", T)
    _i32(ctx.req_of_token, "req_of_token", T)
    _lib.call("core", "pi_latent_kv_write", _ptr(cq_out), _rows(cq_out, "query latent") if cq_out is not None else 0,
              PI_F32 if dtype == torch.float32 else PI_BF16, None if pieces is not None else proj.data_ptr(),
              pieces.N if pieces is not None else _rows(proj, "projection"), _ptr(w_q), w_kv.data_ptr(), _ptr(table),
              ctx.positions.data_ptr(), ctx.req_of_token.data_ptr(), float(eps), T, q_rank, kv_rank, rot, v_rows, _ptr(k_cache),
              _ptr(v_cache), _ptr(block_table), block_table.shape[1] if k_cache is not None else 0, page_size, pages,
              pieces.part.data_ptr() if pieces is not None else None, pieces.splits if pieces is not None else 0,
              pieces.M * pieces.N if pieces is not None else 0, _stream())


def head_gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, heads: int, a_head: Optional[int] = None,
              out_head: Optional[int] = None, rot: int = 0, table: Optional[torch.Tensor] = None,
              w_rows: Optional[torch.Tensor] = None) -> None:
    """A product per head: ``out[t, h * out_head + n] = sum_k a[t, h * a_head + k] * w[h, k, n]`` with ``w``
    [heads, K, N] (a head's matrix stored with its inputs as rows), float32 sums.  ``a_head`` / ``out_head``: the
    distance between two heads in a row of ``a`` / ``out`` (default K + rot / N + rot).  ``rot`` > 0: the ``rot`` numbers
    behind a head's K inputs are turned by the token's angles (``table``: the step's [T, rot] cosines and sines,
    neighbouring pairs) and placed behind the head's N results.  ``w_rows``: the same matrices stored [heads, N, K]
    (a head's outputs as rows), which the matrix-core kernel reads for steps of many tokens (bfloat16)."""
    _gpu(out, a, w, table, w_rows)
    if w.dim() != 3 or w.shape[0] != heads or not w.is_contiguous():
        raise KernelError(f"head product: weights must be contiguous [{heads}, K, N], got {tuple(w.shape)}")
    K, N = int(w.shape[1]), int(w.shape[2])
    a_head = K + rot if a_head is None else int(a_head)
    out_head = N + rot if out_head is None else int(out_head)
    M = a.shape[0]
    if a.dim() != 2 or out.dim() != 2 or out.shape[0] != M or a.dtype != out.dtype or w.dtype != a.dtype:
        raise KernelError(f"head product: a {tuple(a.shape)} {a.dtype}, w {w.dtype}, out {tuple(out.shape)} {out.dtype} do not agree")
    if a.shape[1] < (heads - 1) * a_head + K + rot or out.shape[1] < (heads - 1) * out_head + N + rot:
        raise KernelError(f"head product: rows of {a.shape[1]} / {out.shape[1]} numbers do not hold {heads} heads of {a_head} / {out_head}")
    if rot and (table is None or table.shape != (M, rot) or table.dtype != torch.float32 or not table.is_contiguous()):
        raise KernelError(f"head product: cos / sin table must be contiguous float32 [{M}, {rot}]")
    if M == 0:
        return
    skip = 0
    if _FAST and a.dtype == torch.bfloat16 and w_rows is not None:
        if w_rows.shape != (heads, N, K) or w_rows.dtype != a.dtype or not w_rows.is_contiguous():
            raise KernelError(f"head product: the row-major weights must be contiguous [{heads}, {N}, {K}] {a.dtype}")
        from . import fast
        if fast.head_gemm(out, a, w_rows, heads, K, N, a_head, out_head, _rows(a, "head product a"), _rows(out, "head product out")):
            if rot == 0:
                return
            skip = 1          # the rotated tails are still to make
    _lib.call("core", "pi_head_gemm", out.data_ptr(), _rows(out, "head product out"), out_head, a.data_ptr(), _rows(a, "head product a"),
              a_head, w.data_ptr(), _dt(a), M, heads, K, N, int(rot), _ptr(table), skip, _stream())


# ----------------------------------------------------------------------------- matrix memory
MATRIX_MEMORY_COLUMNS = 16     # value columns per wave of the scan; n and m are kept once per such group


def matrix_memory_state_floats(heads: int, key_dim: int, value_dim: int) -> int:
    """Floats of one request's state: S [heads, d, dv], then (n, m) [heads, slices, d + 1]."""
    slices = -(-value_dim // MATRIX_MEMORY_COLUMNS)
    return heads * key_dim * value_dim + heads * slices * (key_dim + 1)


def matrix_memory_scan(out: torch.Tensor, proj: torch.Tensor, offsets, i_bias: torch.Tensor, f_bias: torch.Tensor, cap: float,
                       q_scale: float, ctx, state: torch.Tensor, heads: int, key_dim: int, value_dim: int) -> None:
    """The matrix-memory recurrence over the step's tokens, request by request, from and into the
    requests' state rows (``state`` float32 [slots, floats], rows ``ctx.slots``).  ``proj`` float32
    rows hold q, k, v and the two gates' pre-activations at column ``offsets`` = (q, k, v, i, f);
    ``out`` float32 [T, heads * value_dim] gets the cell's output before its head norm."""
    _gpu(out, proj, i_bias, f_bias, state)
    T = out.shape[0]
    if out.dtype != torch.float32 or not out.is_contiguous() or out.shape[1] != heads * value_dim:
        raise KernelError(f"matrix memory: output must be contiguous float32 [{T}, {heads * value_dim}]")
    need = max(offsets[0] + heads * key_dim, offsets[1] + heads * key_dim, offsets[2] + heads * value_dim, offsets[3] + heads, offsets[4] + heads)
    if proj.dtype != torch.float32 or proj.dim() != 2 or proj.shape[0] != T or proj.shape[1] < need:
        raise KernelError(f"matrix memory: projection must be float32 [{T}, >= {need}], got {proj.dtype} {tuple(proj.shape)}")
    _f32_vector(i_bias, heads, "matrix memory input-gate bias")
    _f32_vector(f_bias, heads, "matrix memory forget-gate bias")
    floats = matrix_memory_state_floats(heads, key_dim, value_dim)
    if state.dtype != torch.float32 or state.dim() != 2 or not state.is_contiguous() or state.shape[1] < floats:
        raise KernelError(f"matrix memory: state must be contiguous float32 [slots, >= {floats}], got {state.dtype} {tuple(state.shape)}")
    _i32(ctx.q_start, "q_start", ctx.R + 1)
    _i32(ctx.slots, "slots", ctx.R)
    # a request that brings more than one segment of tokens is walked in segments side by side, which
    # needs scratch memory; the most tokens of a request is a host-side number of the step (1 in a
    # step of single tokens, so a replayed decode step never takes this path)
    longest = int(getattr(ctx, "max_q_len", 0) or T)
    lib = _lib.load("core")
    lib.pi_matrix_memory_work_floats.restype = ctypes.c_long
    floats = int(lib.pi_matrix_memory_work_floats(T, ctx.R, longest, heads, key_dim, value_dim))
    work = torch.empty(floats, dtype=torch.float32, device=out.device) if floats else None
    _lib.call("core", "pi_matrix_memory_scan", out.data_ptr(), _rows(out, "out"), proj.data_ptr(), _rows(proj, "projection"),
              int(offsets[0]), int(offsets[1]), int(offsets[2]), int(offsets[3]), int(offsets[4]), i_bias.data_ptr(),
              f_bias.data_ptr(), float(cap), float(q_scale), ctx.q_start.data_ptr(), ctx.slots.data_ptr(), ctx.R,
              state.data_ptr(), state.shape[1], state.shape[0], heads, key_dim, value_dim, T, longest, _ptr(work), floats, _stream())


def head_norm_gate(y: torch.Tensor, o: torch.Tensor, gates: torch.Tensor, weight: torch.Tensor, eps: float, heads: int, value_dim: int,
                   mult: float = 1.0, gate: str = "sigmoid") -> None:
    """y[t, h, :] = mult * o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * weight[h, :] * act(gates[t, h, :]), ``gate``
    naming act: "sigmoid", or "silu" (z * sigmoid(z))."""
    if gate not in ("sigmoid", "silu"):
        raise KernelError(f"head norm: gate activation '{gate}' is not known (sigmoid, silu)")
    _gpu(y, o, gates, weight)
    T, N = y.shape[0], heads * value_dim
    if tuple(y.shape) != (T, N) or not y.is_contiguous():
        raise KernelError(f"head norm: output must be contiguous [{T}, {N}]")
    for t, what in ((o, "input"), (gates, "gates")):
        if t.dtype != torch.float32 or t.dim() != 2 or t.shape[0] != T or t.shape[1] < N:
            raise KernelError(f"head norm: {what} must be float32 [{T}, >= {N}]")
    _f32_vector(weight, N, "head norm weight")
    _lib.call("core", "pi_head_norm_gate", y.data_ptr(), _dt(y), o.data_ptr(), _rows(o, "o"), gates.data_ptr(), _rows(gates, "gates"),
              weight.data_ptr(), float(eps), T, heads, value_dim, float(mult), int(gate == "silu"), _stream())


# ----------------------------------------------------------------------------- routed experts
def route(logits: torch.Tensor, top: int, groups: int = 1, keep: int = 1, renorm: bool = False,
          correction: Optional[torch.Tensor] = None, renorm_eps: float = 0.0):
    """Choose ``top`` experts per row of float32 router logits: (ids int32 [T, top], weights float32
    [T, top]).  Scores are the softmax over all experts; with ``groups`` > 1 only experts of the
    ``keep`` groups with the largest best score may be chosen; weights are the chosen scores
    (divided by their sum + ``renorm_eps`` when ``renorm``).  ``correction`` (float32 [E]): the choice goes
    by score + correction, the weights by the scores alone."""
    _gpu(logits, correction)
    T, E = logits.shape
    _f32_vector(correction, E, "routing correction")
    if logits.dtype != torch.float32:
        raise KernelError("routing: logits must be float32")
    ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    _lib.call("core", "pi_route", ids.data_ptr(), weights.data_ptr(), logits.data_ptr(), _rows(logits, "router logits"), T, E,
              int(top), int(groups), int(keep), int(bool(renorm)), _ptr(correction), float(renorm_eps), _stream())
    return ids, weights


class ExpertRows:
    """A step's (token, choice) entries in expert order, and the tiles of the grouped products
    (``tile`` rows at most, none straddling two experts)."""

    def __init__(self, row_entry, entry_row, tile_expert, tile_row0, tile_rows, top, tile):
        self.row_entry, self.entry_row = row_entry, entry_row
        self.tile_expert, self.tile_row0, self.tile_rows, self.top, self.tile = tile_expert, tile_row0, tile_rows, top, tile

    @property
    def rows(self) -> int:
        return self.row_entry.numel()


def grouped_tile_rows(dtype: torch.dtype) -> int:
    """Rows per tile of the grouped products that serve ``dtype``: the matrix-core kernel's block
    tile for bfloat16, the general kernel's otherwise."""
    if _FAST and dtype == torch.bfloat16 and _lib.build.MODULES["bf16"]:
        return int(_lib.load("bf16").pi_gemm_mfma_group_tile_rows())
    return int(_lib.load("core").pi_group_tile_rows())


def group_entries(ids: torch.Tensor, num_experts: int, tile: Optional[int] = None) -> ExpertRows:
    """Sort the entries of ``ids`` (int32 [T, top]) by expert, on the device.  Entries whose id is ``num_experts``
    or more (identity experts) get no row and no tile."""
    _gpu(ids)
    _i32(ids, "expert ids")
    N = ids.numel()
    tile = int(tile or _lib.load("core").pi_group_tile_rows())
    max_tiles = -(-N // tile) + num_experts
    meta = torch.empty(2 * N + 3 * max_tiles, dtype=torch.int32, device=ids.device)
    row_entry, entry_row = meta[:N], meta[N:2 * N]
    te, t0, tr = (meta[2 * N + i * max_tiles: 2 * N + (i + 1) * max_tiles] for i in range(3))
    _lib.call("core", "pi_group_entries", ids.data_ptr(), N, int(num_experts), row_entry.data_ptr(), entry_row.data_ptr(),
              te.data_ptr(), t0.data_ptr(), tr.data_ptr(), max_tiles, tile, _stream())
    return ExpertRows(row_entry, entry_row, te, t0, tr, ids.shape[1], tile)


def gather_rows(src: torch.Tensor, rows: ExpertRows) -> torch.Tensor:
    """The tokens' activations copied into expert order: [entries, D]."""
    _gpu(src)
    if src.dim() != 2 or not src.is_contiguous():
        raise KernelError("gather: activations must be contiguous 2-D")
    out = torch.empty((rows.rows, src.shape[1]), dtype=src.dtype, device=src.device)
    _lib.call("core", "pi_gather_rows", out.data_ptr(), src.data_ptr(), _dt(src), rows.row_entry.data_ptr(), rows.rows, rows.top,
              src.shape[1], _stream())
    return out


def _grouped_fast(out, a, w, rows: ExpertRows, epilogue: int) -> bool:
    """The matrix-core grouped product, when the operands are what it takes."""
    if not (_FAST and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and _lib.build.MODULES["bf16"]):
        return False
    K = w.shape[2]
    if K % 8 or _rows(a, "a") % 8 or a.data_ptr() % 16 or w.data_ptr() % 16 or (w.shape[1] * K) % 8:
        return False
    if rows.tile != int(_lib.load("bf16").pi_gemm_mfma_group_tile_rows()):
        return False
    _lib.call("bf16", "pi_gemm_mfma_grouped", out.data_ptr(), epilogue, _rows(out, "out"), a.data_ptr(), _rows(a, "a"), w.data_ptr(),
              K, w.shape[1] * K, rows.tile_expert.data_ptr(), rows.tile_row0.data_ptr(), rows.tile_rows.data_ptr(),
              rows.tile_expert.numel(), w.shape[1], K, 0, 0, _stream())
    return True


def grouped_gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, rows: ExpertRows) -> None:
    """out[row] = a[row] @ w[expert of row]^T for rows in expert order; ``w`` is [experts, N, K]."""
    _gpu(out, a, w)
    if w.dim() != 3 or not w.is_contiguous() or a.shape != (rows.rows, w.shape[2]) or out.shape != (rows.rows, w.shape[1]):
        raise KernelError(f"grouped product: shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    if a.dtype != w.dtype:
        raise KernelError(f"grouped product: activations {a.dtype} and weights {w.dtype} must have one type")
    if rows.rows == 0:
        return
    if out.dtype in (torch.bfloat16, torch.float32) and _grouped_fast(out, a, w, rows, 0 if out.dtype == torch.bfloat16 else 1):
        return
    _lib.call("core", "pi_grouped_gemm_general", out.data_ptr(), _dt(out), _rows(out, "out"), a.data_ptr(), _dt(a), _rows(a, "a"),
              w.data_ptr(), _dt(w), w.shape[2], w.shape[1] * w.shape[2], rows.tile_expert.data_ptr(), rows.tile_row0.data_ptr(),
              rows.tile_rows.data_ptr(), rows.tile_expert.numel(), w.shape[1], w.shape[2], _stream())


def grouped_gemm_swiglu(out: torch.Tensor, a: torch.Tensor, w_gate_up: torch.Tensor, rows: ExpertRows, block: int = 0) -> None:
    """out[row] = silu(a[row] @ Wg^T) * (a[row] @ Wu^T) with the row's expert's matrices: ``w_gate_up``
    [experts, 2F, K] holds every expert's gate and up rows in halves (``block`` 0) or interleaved in
    blocks of ``block`` rows.  With bfloat16 operands and blocks of 16 product and activation are one kernel."""
    _gpu(out, a, w_gate_up)
    F2 = w_gate_up.shape[1]
    if out.shape != (rows.rows, F2 // 2) or out.dtype != a.dtype:
        raise KernelError(f"grouped swiglu: out {tuple(out.shape)} does not match {rows.rows} x {F2 // 2}")
    if rows.rows == 0:
        return
    if block == 16 and F2 % 32 == 0 and out.is_contiguous() and _grouped_fast(out, a, w_gate_up, rows, 3):
        return
    gu = torch.empty((rows.rows, F2), dtype=a.dtype, device=a.device)
    grouped_gemm(gu, a, w_gate_up, rows)
    swiglu(out, gu, block)


def grouped_gemm_relu_squared(out: torch.Tensor, a: torch.Tensor, w_up: torch.Tensor, rows: ExpertRows) -> None:
    """out[row] = max(a[row] @ W^T, 0)^2 with the row's expert's matrix; ``w_up`` is [experts, F, K].  The square is taken on
    the product's float32 result."""
    _gpu(out, a, w_up)
    if out.shape != (rows.rows, w_up.shape[1]):
        raise KernelError(f"grouped squared relu: out {tuple(out.shape)} does not match {rows.rows} x {w_up.shape[1]}")
    if rows.rows == 0:
        return
    if out.dtype == torch.bfloat16 and out.is_contiguous() and _grouped_fast(out, a, w_up, rows, EPI_RELU2):
        return
    u = torch.empty((rows.rows, w_up.shape[1]), dtype=torch.float32, device=a.device)
    grouped_gemm(u, a, w_up, rows)
    relu_squared(out, u)


def combine_choices(out: torch.Tensor, y: torch.Tensor, weights: torch.Tensor, rows: ExpertRows, accumulate: bool = False,
                    ids: Optional[torch.Tensor] = None, num_real: int = 0, h: Optional[torch.Tensor] = None) -> None:
    """out[t] (+)= sum over the token's choices of weight * y[row of (t, choice)], in choice order (float32).
    With ``ids`` (int32 [T, top]), ``num_real`` and the tokens' activations ``h`` [T, D]: a choice whose id is
    ``num_real`` or more is an identity expert and contributes weight * h[t]."""
    _gpu(out, y, weights, ids, h)
    if ids is not None:
        _i32(ids, "expert ids", weights.numel())
        if h is None or h.shape != out.shape or not h.is_contiguous():
            raise KernelError("combine: identity experts need the tokens' activations, contiguous and as wide as the output")
    T, D = out.shape
    if out.dtype != torch.float32 or y.dtype != torch.float32 or not (out.is_contiguous() and y.is_contiguous()) or y.shape != (rows.rows, D):
        raise KernelError(f"combine: expected float32 out [{T}, {D}] and y [{rows.rows}, {D}]")
    if weights.dtype != torch.float32 or not weights.is_contiguous() or weights.numel() != rows.rows:
        raise KernelError("combine: one float32 weight per entry is needed")
    _lib.call("core", "pi_combine_choices", out.data_ptr(), y.data_ptr(), weights.data_ptr(), rows.entry_row.data_ptr(), T, rows.top, D,
              int(bool(accumulate)), _ptr(ids), int(num_real), _ptr(h), _dt(h) if h is not None else PI_F32, _stream())


# ----------------------------------------------------------------------------- mixers with a state of fixed size
CONV_MAX_TAPS = 8


def _state_rows(state: torch.Tensor, floats: int, what: str) -> None:
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < floats or not state.is_cuda:
        raise KernelError(f"{what}: state must be float32 [slots, >= {floats}] with dense rows on the GPU, got {state.dtype} {tuple(state.shape)}")


def _f32_rows(t: torch.Tensor, T: int, cols: int, what: str) -> int:
    if t.dtype != torch.float32 or t.dim() != 2 or t.shape[0] != T or t.shape[1] < cols:
        raise KernelError(f"{what}: expected float32 [{T}, >= {cols}], got {t.dtype} {tuple(t.shape)}")
    return _rows(t, what)


SCAN_COLUMNS = 16        # value columns of a block of the state walks: four waves of four columns


def _scan_rows_per_lane(rows: int) -> int:
    nr = next((n for n in (1, 2, 4, 8, 16) if 16 * n >= rows), 0)
    if nr == 0 or rows <= 0:
        raise KernelError(f"state walk: {rows} rows per head are not within 1 .. 256")
    return nr


def scan_state_floats(heads: int, rows: int, cols: int) -> int:
    """Floats of one request's state [heads, rows, cols] as the state walks keep it: in their own order,
    [head][slice of 16 columns][wave][i][lane], where lane = 16 * column + part of wave w holds row
    part * NR + i of column 16 * slice + 4 * w + column (NR: the rows per lane, the power of two up to 16 with
    16 * NR >= rows), padded to whole slices and rows."""
    return int(heads) * -(-int(cols) // SCAN_COLUMNS) * 4 * _scan_rows_per_lane(rows) * 64     # the kernels' own count: pi_scan_state_floats


def unpack_scan_state(row: torch.Tensor, heads: int, rows: int, cols: int) -> torch.Tensor:
    """One request's state as [heads, rows, cols], from the walks' own order (for tests and inspection)."""
    floats, nr, slices = scan_state_floats(heads, rows, cols), _scan_rows_per_lane(rows), -(-cols // SCAN_COLUMNS)
    t = row[:floats].view(heads, slices, 4, nr, 4, 16)               # [h, z, wave, i, column, part]
    t = t.permute(0, 5, 3, 1, 2, 4).reshape(heads, 16 * nr, slices * SCAN_COLUMNS)   # row = part * nr + i, col = z * 16 + wave * 4 + column
    return t[:, :rows, :cols]


def causal_conv_silu(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], ctx,
                     state: torch.Tensor) -> None:
    """out[t, c] = silu(bias[c] + sum_j weight[c, j] * x[t - (taps - 1) + j, c]) within each request of the
    step; the inputs before a request's first token of this step come from its state row
    (``state`` float32 [slots, >= (taps - 1) * C], laid out [taps - 1, C], rows ``ctx.slots``), which
    then takes the request's last taps - 1 inputs.  ``x`` and ``out`` are float32 [T, >= C] (column
    views of wider tensors are fine; not in place)."""
    _gpu(out, x, weight, bias, state)
    T = x.shape[0]
    C, taps = weight.shape
    if taps > CONV_MAX_TAPS:
        raise KernelError(f"convolution: {taps} taps are more than {CONV_MAX_TAPS}")
    if not weight.is_contiguous() or (bias is not None and (bias.shape != (C,) or bias.dtype != weight.dtype or not bias.is_contiguous())):
        raise KernelError(f"convolution: weight must be contiguous [{C}, {taps}] and bias [{C}] of the same type")
    ldx, ldo = _f32_rows(x, T, C, "convolution input"), _f32_rows(out, T, C, "convolution output")
    _state_rows(state, (taps - 1) * C, "convolution")
    _i32(ctx.q_start, "q_start", ctx.R + 1)
    _i32(ctx.slots, "slots", ctx.R)
    longest = int(getattr(ctx, "max_q_len", 0) or T)
    _lib.call("core", "pi_causal_conv_silu", out.data_ptr(), ldo, x.data_ptr(), ldx, weight.data_ptr(), _ptr(bias), _dt(weight), C, taps,
              ctx.q_start.data_ptr(), ctx.slots.data_ptr(), ctx.R, longest, state.data_ptr(), state.stride(0), _stream())


def state_space_scan(y: torch.Tensor, xbc: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor,
                     skip: torch.Tensor, ctx, state: torch.Tensor, heads: int, value_dim: int, state_dim: int, groups: int) -> None:
    """The state-space recurrence over the step's tokens, request by request, from and into the
    requests' state rows (``state`` float32 [slots, >= scan_state_floats(heads, state_dim, value_dim)], rows ``ctx.slots``):
    ``S <- exp(-exp(a_log) * dt') S + dt' B x^T``, ``y = S^T C + skip * x`` with ``dt' = softplus(dt + dt_bias)``.
    ``xbc`` float32 rows hold x [heads * value_dim], B and C [groups * state_dim each]; ``dt`` float32 [T, heads]
    (a column view is fine); ``y`` float32 [T, heads * value_dim]."""
    _gpu(y, xbc, dt, dt_bias, a_log, skip, state)
    T, inner = y.shape[0], heads * value_dim
    ldy = _f32_rows(y, T, inner, "state space output")
    ldx = _f32_rows(xbc, T, inner + 2 * groups * state_dim, "state space input")
    ldd = _f32_rows(dt, T, heads, "state space steps")
    for t, what in ((dt_bias, "step bias"), (a_log, "decay"), (skip, "skip")):
        _f32_vector(t, heads, f"state space {what}")
    _state_rows(state, scan_state_floats(heads, state_dim, value_dim), "state space")
    _i32(ctx.q_start, "q_start", ctx.R + 1)
    _i32(ctx.slots, "slots", ctx.R)
    _lib.call("core", "pi_state_space_scan", y.data_ptr(), ldy, xbc.data_ptr(), ldx, dt.data_ptr(), ldd, dt_bias.data_ptr(),
              a_log.data_ptr(), skip.data_ptr(), ctx.q_start.data_ptr(), ctx.slots.data_ptr(), ctx.R,
              int(getattr(ctx, "max_q_len", 0) or T), state.data_ptr(), state.stride(0), heads, value_dim, state_dim, groups, _stream())


def gated_group_norm(out: torch.Tensor, y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, eps: float, parts: int,
                     mult: float = 1.0) -> None:
    """out = mult * weight * v / sqrt(mean(v^2) + eps) with v = y * silu(z), the mean taken over each
    of ``parts`` equal parts of a row.  ``y``, ``z`` float32 [T, >= N]; ``out`` [T, N] in any type."""
    _gpu(out, y, z, weight)
    T, N = out.shape
    if N % parts:
        raise KernelError(f"gated norm: {N} columns do not split into {parts} parts")
    _f32_vector(weight, N, "gated norm weight")
    _lib.call("core", "pi_gated_group_norm", out.data_ptr(), _dt(out), _rows(out, "gated norm out"), y.data_ptr(),
              _f32_rows(y, T, N, "gated norm input"), z.data_ptr(), _f32_rows(z, T, N, "gated norm gate"), weight.data_ptr(),
              float(eps), float(mult), T, N, int(parts), _stream())


SCAN_KINDS = {"channel_delta": 0, "head_delta": 1, "decayed_outer": 2}


def delta_scan(o: torch.Tensor, qkv: torch.Tensor, a: torch.Tensor, dt_bias: torch.Tensor, a_log: Optional[torch.Tensor],
               b: Optional[torch.Tensor], ctx, state: torch.Tensor, heads: int, kv_heads: int, key_dim: int, value_dim: int,
               q_scale: float, unit_eps: float, kind: str = "channel_delta", tau: float = 1.0) -> None:
    """The gated delta rule with a decay per head and key channel over the step's tokens, from and
    into the requests' state rows (``state`` float32 [slots, >= scan_state_floats(heads, key_dim, value_dim)]):
    ``S <- diag(decay) S; u = beta (v - S^T k^); S <- S + k^ u^T; o = S^T q^`` with unit vectors
    ``k^``, ``q^`` (the latter times ``q_scale``), ``decay = exp(-exp(a_log) * softplus(a + dt_bias))``,
    ``beta = sigmoid(b)``.  ``qkv``, ``a`` and ``b`` are CHANGED IN PLACE: a first kernel turns them into the unit
    vectors, the decays and beta, once per token and head, before the walk reads them.  ``qkv`` float32 rows hold q and k [kv_heads * key_dim each] and v
    [heads * value_dim]; ``a`` float32 [T, heads * key_dim]; ``b`` float32 [T, heads] (a column view
    is fine); ``o`` float32 [T, heads * value_dim].

    ``kind`` "head_delta": the same with one decay per head, ``S <- decay S``: ``a`` is [T, heads] and ``dt_bias`` [heads].
    ``kind`` "decayed_outer" (gated linear attention): ``S <- diag(decay) S + k v^T; o = S^T (q * q_scale)`` with
    ``decay = sigmoid(a + dt_bias)^(1 / tau)`` per head and key channel; no unit vectors, no ``b``, no ``a_log``."""
    if kind not in SCAN_KINDS:
        raise KernelError(f"state walk: kind '{kind}' is not known ({', '.join(SCAN_KINDS)})")
    _gpu(o, qkv, a, dt_bias, a_log, b, state)
    T = o.shape[0]
    per_head = kind == "head_delta"
    outer = kind == "decayed_outer"
    ldo = _f32_rows(o, T, heads * value_dim, "delta rule output")
    ldq = _f32_rows(qkv, T, 2 * kv_heads * key_dim + heads * value_dim, "delta rule input")
    lda = _f32_rows(a, T, heads if per_head else heads * key_dim, "delta rule decays")
    ldb = 0 if outer else _f32_rows(b, T, heads, "delta rule beta")
    _f32_vector(dt_bias, heads if per_head else heads * key_dim, "delta rule decay bias")
    if not outer:
        _f32_vector(a_log, heads, "delta rule decay rate")
    elif not tau > 0.0:
        raise KernelError(f"state walk: the root taken of the decays must be positive, got {tau}")
    _state_rows(state, scan_state_floats(heads, key_dim, value_dim), "delta rule")
    _i32(ctx.q_start, "q_start", ctx.R + 1)
    _i32(ctx.slots, "slots", ctx.R)
    _lib.call("core", "pi_delta_scan", o.data_ptr(), ldo, qkv.data_ptr(), ldq, a.data_ptr(), lda, dt_bias.data_ptr(), _ptr(a_log),
              _ptr(b), ldb, ctx.q_start.data_ptr(), ctx.slots.data_ptr(), ctx.R, T, int(getattr(ctx, "max_q_len", 0) or T), state.data_ptr(), state.stride(0), heads,
              kv_heads, key_dim, value_dim, float(q_scale), float(unit_eps), SCAN_KINDS[kind], float(tau), _stream())


def clamped_glu(out: torch.Tensor, gate_up: torch.Tensor, gate_bias: torch.Tensor, up_bias: Optional[torch.Tensor], limit: float,
                alpha: float, x: Optional[torch.Tensor] = None, x_bias: Optional[torch.Tensor] = None, block: int = 0) -> None:
    """out = g * sigmoid(alpha * g) * (u + 1) with g = min(gate + gate_bias, limit) and
    u = clamp(up + up_bias, -limit, limit).  ``block`` = 0: ``gate_up`` [T, 2I] holds the two products in halves;
    ``block`` = b: gate and up interleaved in blocks of b columns, and ``gate_bias`` [2I] holds both biases in the
    same order (``up_bias`` None).  With ``x`` (the float32 stream) and ``x_bias``: x[t, :] += x_bias as well, the
    bias of the product that follows."""
    _gpu(out, gate_up, gate_bias, up_bias, x, x_bias)
    T, I = out.shape
    if gate_up.shape != (T, 2 * I) or not (out.is_contiguous() and gate_up.is_contiguous()):
        raise KernelError(f"clamped unit: expected contiguous gate_up [{T}, {2 * I}], got {tuple(gate_up.shape)}")
    if block < 0 or (block and (I % block or up_bias is not None or gate_bias.numel() != 2 * I)):
        raise KernelError(f"clamped unit: interleave block {block} needs {I} % block == 0 and one bias vector of {2 * I}")
    biases = [gate_bias] + ([up_bias] if not block else []) + ([x_bias] if x is not None else [])
    if any(b is None or b.dtype != gate_bias.dtype or not b.is_contiguous() for b in biases) or (not block and (gate_bias.numel() != I or up_bias.numel() != I)):
        raise KernelError(f"clamped unit: biases must be contiguous [{I}] of one type")
    D = 0
    if x is not None:
        D = x.shape[1]
        if x.dtype != torch.float32 or not x.is_contiguous() or x.shape[0] != T or x_bias is None or x_bias.numel() != D:
            raise KernelError(f"clamped unit: the stream must be contiguous float32 [{T}, D] with a bias [D]")
    _lib.call("core", "pi_clamped_glu", out.data_ptr(), _dt(out), gate_up.data_ptr(), _dt(gate_up), gate_bias.data_ptr(),
              _ptr(up_bias), _ptr(x_bias) if x is not None else None, _dt(gate_bias), float(limit), float(alpha), T, I,
              _ptr(x), D, int(block), _stream())


def add_row_bias(x: torch.Tensor, bias: torch.Tensor) -> None:
    """x[t, :] += bias (the float32 stream; the bias in float32)."""
    _gpu(x, bias)
    T, D = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous() or bias.dtype != torch.float32 or not bias.is_contiguous() or bias.numel() != D:
        raise KernelError(f"row bias: expected a contiguous float32 stream [{T}, {D}] and a float32 bias [{D}]")
    _lib.call("core", "pi_clamped_glu", None, PI_F32, None, PI_F32, None, None, bias.data_ptr(), PI_F32, 0.0, 0.0, T, 0,
              x.data_ptr(), D, 0, _stream())


def gemm_clamped_glu(out: torch.Tensor, a: torch.Tensor, w_gate_up: torch.Tensor, bias: torch.Tensor, limit: float, alpha: float,
                     block: int, ws: Optional[KernelWorkspace] = None, x: Optional[torch.Tensor] = None,
                     x_bias: Optional[torch.Tensor] = None) -> None:
    """out[M, I] = the clamped gated unit (``clamped_glu``) of a @ w_gate_up^T + bias, where ``w_gate_up`` [2I, K] and
    ``bias`` (float32 [2I]) hold gate and up rows in halves (``block`` 0) or interleaved in blocks of ``block``.  With
    bfloat16 operands, blocks of 16 and more rows than the weight-streaming products take, product and unit are
    one kernel; otherwise the product's float32 result goes through the unit's own kernel.  ``x`` and ``x_bias``
    (float32): the stream's rows get ``x_bias`` added on the way (the bias of the product that follows), by the unit's
    kernel where it runs, by a kernel of its own otherwise; an update of ``x`` that is pending in ``ws`` is applied first."""
    _gpu(out, a, w_gate_up, bias)
    if x is not None:
        materialize(x, ws)
    M, I = out.shape
    if w_gate_up.shape[0] != 2 * I or a.shape != (M, w_gate_up.shape[1]) or bias.dtype != torch.float32 or bias.numel() != 2 * I:
        raise KernelError(f"gemm_clamped_glu: shapes do not agree: a {tuple(a.shape)}, w {tuple(w_gate_up.shape)}, out {tuple(out.shape)}")
    if M == 0:
        return
    if _FAST and block == 16 and a.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and out.is_contiguous() and bias.is_contiguous():
        from . import fast
        if fast.gemm_clamped_glu(out, a, w_gate_up, bias, limit, alpha, M, 2 * I, a.shape[1], _rows(a, "gemm a"), _rows(w_gate_up, "gemm w")):
            if ws is not None:
                ws.counts["gated_epilogues"] += 1
            if x is not None:
                add_row_bias(x, x_bias)
            return
    gu = torch.empty((M, 2 * I), dtype=torch.float32, device=a.device)
    gemm(gu, a, w_gate_up, ws=ws)
    if block:
        clamped_glu(out, gu, bias, None, limit, alpha, x, x_bias, block=block)
    else:
        clamped_glu(out, gu, bias[:I], bias[I:], limit, alpha, x, x_bias)
