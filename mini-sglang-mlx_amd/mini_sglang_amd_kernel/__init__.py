"""MI355X counterpart of the reference's ``mini_sglang_mlx_kernel`` module, for the
paged-attention path only.

Same function names, positional order and keyword names as the nanobind module
(mini-sglang-mlx-kernel/csrc/bindings.cpp:27-55, mini_sglang_mlx_kernel/__init__.py:1-9);
``mx.array`` becomes ``torch.Tensor`` on a ROCm device.  Every call is an eager,
stream-ordered launch of hand-written gfx950 kernels through the C ABI of
``include/msgl_paged_attention.h``; nothing synchronises with the host and there is no
other implementation to fall back to.

Argument errors raise ``RuntimeError`` with the reference's message text
(paged_decode_attention.cpp:25-62, paged_prefill_attention.cpp:31-76,
store_kv_cache.cpp:22-63).
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from . import _lib

__all__ = ["store_kv_cache", "paged_decode_attention", "paged_prefill_attention",
           "build_attention_metadata", "qk_norm_rope_store", "gdn_state_inplace",
           "fast_compare_key"]

_DTYPE_CODE = {torch.bfloat16: _lib.MSGL_DTYPE_BF16, torch.float16: _lib.MSGL_DTYPE_F16}


def _fail(op: str, msg: str):
    raise RuntimeError(f"{op}: {msg}")


_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(stream, device) -> int:
    if stream is not None:
        return int(stream.cuda_stream)
    if _raw_current_stream is not None:  # the handle without building a Stream object
        return int(_raw_current_stream(device.index if device.index is not None
                                       else torch.cuda.current_device()))
    return int(torch.cuda.current_stream(device).cuda_stream)


class _on_device:
    """``torch.cuda.device(dev)`` that costs nothing when ``dev`` is current already (the usual
    case: one process per GPU), and, for a call with an explicit ``stream=``, that stream made
    torch's current one for the duration of the call.  The second part is what makes a foreign
    stream safe: the output, the workspace and any ``.contiguous()`` copy of an argument are
    then allocated and produced on the stream the kernels run on, so torch's caching allocator
    never hands one of these blocks to work that is still in flight on another stream."""

    __slots__ = ("_guards",)

    def __init__(self, dev: torch.device, stream=None):
        self._guards = []
        index = dev.index
        if index is not None and index != torch.cuda.current_device():
            self._guards.append(torch.cuda.device(dev))
        if stream is not None:
            if not isinstance(stream, torch.cuda.Stream):
                stream = torch.cuda.ExternalStream(int(stream.cuda_stream), device=dev)
            self._guards.append(torch.cuda.stream(stream))

    def __enter__(self):
        for g in self._guards:
            g.__enter__()

    def __exit__(self, *exc):
        for g in reversed(self._guards):
            g.__exit__(*exc)
        return False


def _require_device(op: str, *tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        _fail(op, "tensors must live on a ROCm GPU device (no CPU implementation exists)")
    for t in tensors:
        if t.device != dev:
            _fail(op, "all tensors must be on the same device")
    return dev


def _pool_stride0(op: str, pool: torch.Tensor, name: str) -> int:
    if pool.stride(2) != 1 or pool.stride(1) != pool.shape[2]:
        _fail(op, f"{name} must be contiguous in its (num_kv_heads, head_dim) dimensions")
    # a one-slot pool may report any leading stride
    return pool.stride(0) if pool.shape[0] > 1 else pool.shape[1] * pool.shape[2]


def _int32_1d(op: str, t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.int32:
        _fail(op, f"{name} must be int32")
    return t if t.is_contiguous() else t.contiguous()


def _checks_on(validate: Optional[bool]) -> bool:
    """Index validation is opt-in: ``validate=True`` on the call, or ``MSGL_DEBUG_CHECKS=1`` in
    the environment for every call that does not say ``validate=False``.  It costs a few small
    device reductions and ONE host synchronisation per call, so it is off by default, and it is
    skipped while the current stream is being captured into a graph (a capture cannot sync)."""
    if validate is None:
        validate = os.environ.get("MSGL_DEBUG_CHECKS", "0") not in ("", "0")
    if not validate:
        return False
    return not (torch.cuda.is_available() and torch.cuda.is_current_stream_capturing())


def _validate_slot_ids(op: str, name: str, ids: torch.Tensor, num_slots: int,
                       unique: bool = False) -> None:
    """Every id inside ``[0, num_slots)`` and, for a store, no id twice.  The kernels read or
    write ``pool[id]`` unchecked (a stray id is a wild access: a GPU memory fault, not a wrong
    value; the writers skip such a row, the readers cannot), and two rows stored to one slot
    race (store_kv_cache.metal:24-30 has the same hole; the reference's allocator hands out
    distinct slots, scheduler/cache.py:45-57).  Works on any device: min, max and a sort there,
    then one transfer of three numbers."""
    if ids.numel() == 0:
        return
    lo, hi = torch.aminmax(ids)
    dup = torch.zeros((), dtype=torch.int64, device=ids.device)
    if unique and ids.numel() > 1:
        srt = torch.sort(ids).values
        dup = (srt[1:] == srt[:-1]).sum()
    lo, hi, dup = (int(x) for x in torch.stack([lo.long(), hi.long(), dup]).tolist())
    if lo < 0 or hi >= num_slots:
        _fail(op, f"{name} holds slot ids outside [0, {num_slots}): min {lo}, max {hi}")
    if dup:
        _fail(op, f"{name} holds {dup} duplicate slot id(s); rows stored to one slot race")


def _validate_indptr(op: str, name: str, indptr: torch.Tensor, limit: int, what: str) -> None:
    """A CSR offset array must start at >= 0, never decrease and end inside the array it
    indexes."""
    first, last = indptr[0], indptr[-1]
    down = (indptr[1:] < indptr[:-1]).sum() if indptr.numel() > 1 else torch.zeros_like(first)
    first, last, down = (int(x) for x in torch.stack([first.long(), last.long(), down.long()]).tolist())
    if first < 0 or down:
        _fail(op, f"{name} must start at >= 0 and be non-decreasing")
    if last > limit:
        _fail(op, f"{name} ends at {last}, beyond the {limit} entries of {what}")


def _check_rc(op: str, rc: int) -> None:
    if rc != 0:
        _fail(op, _lib.strerror(rc))


def store_kv_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, indices: torch.Tensor,
                   k: torch.Tensor, v: torch.Tensor, *, stream=None,
                   validate: Optional[bool] = None) -> None:
    """In place: ``k_cache[indices[r]] = k[r]``, ``v_cache[indices[r]] = v[r]`` (bit copy).

    Drop-in for ``mini_sglang_mlx_kernel.store_kv_cache`` (store_kv_cache.cpp:14-107).
    ``indices`` must be unique; duplicates race exactly as in the reference.  A slot id outside
    the pool stores nothing.  ``validate=True`` (or ``MSGL_DEBUG_CHECKS=1``) checks range and
    uniqueness first, at the price of one host synchronisation.
    """
    op = "store_kv_cache"
    if k_cache.dim() != 3 or v_cache.dim() != 3:
        _fail(op, "k_cache and v_cache must be 3D (num_pages, num_kv_heads, head_dim)")
    if indices.dim() != 1:
        _fail(op, "indices must be 1D")
    if k.dim() != 3 or v.dim() != 3:
        _fail(op, "k and v must be 3D (length, num_kv_heads, head_dim)")
    if not (k_cache.dtype == v_cache.dtype == k.dtype == v.dtype):
        _fail(op, "k_cache, v_cache, k, v must have the same dtype")
    if indices.dtype != torch.int32:
        _fail(op, "indices must be int32")
    num_pages, num_kv_heads, head_dim = k_cache.shape
    length = indices.shape[0]
    if head_dim % 4 != 0:
        _fail(op, "head_dim must be a multiple of 4")
    if tuple(v_cache.shape) != (num_pages, num_kv_heads, head_dim):
        _fail(op, "v_cache shape must match k_cache")
    if tuple(k.shape) != (length, num_kv_heads, head_dim) or tuple(v.shape) != tuple(k.shape):
        _fail(op, "k and v shape must be (length, num_kv_heads, head_dim)")
    if k_cache.element_size() not in (2, 4):
        _fail(op, "unsupported dtype, must be float16, bfloat16 or float32")
    dev = _require_device(op, k_cache, v_cache, indices, k, v)
    if length == 0:
        return
    if _checks_on(validate):
        _validate_slot_ids(op, "indices", indices, num_pages, unique=True)
    row = num_kv_heads * head_dim

    def _src(t):
        if t.stride(2) != 1 or t.stride(1) != head_dim:
            t = t.contiguous()
        return t, (t.stride(0) if t.shape[0] > 1 else row)

    with _on_device(dev, stream):
        k, k_stride0 = _src(k)
        v, v_stride0 = _src(v)
        indices = indices if indices.is_contiguous() else indices.contiguous()
        rc = _lib.load().msgl_store_kv_cache(
            k_cache.data_ptr(), v_cache.data_ptr(), indices.data_ptr(), k.data_ptr(),
            v.data_ptr(), length, num_kv_heads, head_dim, num_pages,
            _pool_stride0(op, k_cache, "k_cache"), _pool_stride0(op, v_cache, "v_cache"),
            k_stride0, v_stride0, k_cache.element_size(), _stream_ptr(stream, dev))
    _check_rc(op, rc)


def _attention_dtype(op: str, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     half_ok: bool) -> int:
    if q.dtype not in _DTYPE_CODE:
        _fail(op, "unsupported dtype, must be float16 or bfloat16")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        _fail(op, "q, k_cache and v_cache must have the same dtype")
    if q.dtype != torch.bfloat16 and not half_ok:
        # float16 exists for decode only, as in the reference: its prefill kernel is
        # instantiated for bfloat16 alone (paged_prefill_attention.metal:646-647)
        _fail(op, "unsupported dtype, the prefill kernel is bfloat16 only")
    return _DTYPE_CODE[q.dtype]


def _workspace(nbytes: int, dev) -> Optional[torch.Tensor]:
    """Scratch from torch's caching allocator, taken on the launch stream (see ``_on_device``):
    safe to drop right after the launch because the allocator reuses a block in stream order."""
    if nbytes == 0:
        return None
    return torch.empty(nbytes, dtype=torch.uint8, device=dev)


def paged_decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           kv_indptr: torch.Tensor, kv_indices: torch.Tensor,
                           num_kv_splits: torch.Tensor, sm_scale: float, max_kv_splits: int,
                           *, stream=None, validate: Optional[bool] = None) -> torch.Tensor:
    """GQA paged decode: ``q (batch, n_q, d)`` against the tokens listed in ``kv_indices``.

    Drop-in for ``mini_sglang_mlx_kernel.paged_decode_attention``
    (paged_decode_attention.cpp:15-73).  Returns ``(batch, n_q, d)`` in the dtype of ``q``.
    ``validate=True`` (or ``MSGL_DEBUG_CHECKS=1``) first checks ``kv_indptr`` and that every
    entry of ``kv_indices`` names a slot of the pool (one host synchronisation).
    """
    op = "paged_decode_attention"
    if q.dim() != 3:
        _fail(op, "q must be 3D (batch, num_q_heads, head_dim)")
    if k_cache.dim() != 3 or v_cache.dim() != 3:
        _fail(op, "k_cache and v_cache must be 3D (num_pages, num_kv_heads, head_dim)")
    if kv_indptr.dim() != 1 or kv_indices.dim() != 1 or num_kv_splits.dim() != 1:
        _fail(op, "kv_indptr, kv_indices, num_kv_splits must be 1D")
    batch, num_q_heads, head_dim = q.shape
    num_kv_heads = k_cache.shape[1]
    if head_dim not in (128, 256):
        _fail(op, "head_dim must be 128 or 256")
    if num_q_heads % num_kv_heads != 0:
        _fail(op, "num_q_heads must be a multiple of num_kv_heads")
    if num_q_heads // num_kv_heads > 16:
        _fail(op, "only q_heads/kv_heads <= 16 is supported")
    if k_cache.shape[2] != head_dim or v_cache.shape[2] != head_dim:
        _fail(op, "cache head_dim must match q head_dim")
    if v_cache.shape[1] != num_kv_heads:
        _fail(op, "v_cache shape must match k_cache")
    dtype = _attention_dtype(op, q, k_cache, v_cache, half_ok=True)
    kv_indptr = _int32_1d(op, kv_indptr, "kv_indptr")
    kv_indices = _int32_1d(op, kv_indices, "kv_indices")
    num_kv_splits = _int32_1d(op, num_kv_splits, "num_kv_splits")
    if kv_indptr.shape[0] != batch + 1:
        _fail(op, "kv_indptr must have batch + 1 entries")
    if num_kv_splits.shape[0] != batch:
        _fail(op, "num_kv_splits must have batch entries")
    dev = _require_device(op, q, k_cache, v_cache, kv_indptr, kv_indices, num_kv_splits)
    lib = _lib.load()
    total_kv = kv_indices.shape[0]
    if batch > 0 and _checks_on(validate):
        _validate_indptr(op, "kv_indptr", kv_indptr, total_kv, "kv_indices")
        _validate_slot_ids(op, "kv_indices", kv_indices, k_cache.shape[0])
    with _on_device(dev, stream):
        q = q if q.is_contiguous() else q.contiguous()
        out = torch.empty((batch, num_q_heads, head_dim), dtype=q.dtype, device=dev)
        if batch == 0:
            return out
        ws_bytes = lib.msgl_paged_decode_workspace_bytes(batch, total_kv, num_q_heads,
                                                         num_kv_heads, head_dim)
        ws = _workspace(ws_bytes, dev)
        rc = lib.msgl_paged_decode_attention(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), kv_indptr.data_ptr(),
            kv_indices.data_ptr(), num_kv_splits.data_ptr(), out.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws_bytes, batch, total_kv, num_q_heads,
            num_kv_heads, head_dim, k_cache.shape[0], _pool_stride0(op, k_cache, "k_cache"),
            _pool_stride0(op, v_cache, "v_cache"), float(sm_scale), int(max_kv_splits), dtype,
            _stream_ptr(stream, dev))
    _check_rc(op, rc)
    return out


def paged_prefill_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            qo_indptr: torch.Tensor, kv_indptr: torch.Tensor,
                            kv_indices: torch.Tensor, prefix_lens: torch.Tensor,
                            sm_scale: float, max_len_extend: int, *,
                            is_cross_attention: bool = False, sliding_window_size: int = 0,
                            stream=None, validate: Optional[bool] = None) -> torch.Tensor:
    """Paged extend attention on top of a cached prefix.

    Drop-in for ``mini_sglang_mlx_kernel.paged_prefill_attention``
    (paged_prefill_attention.cpp:18-87).  Query ``i`` of request ``b`` sits at position
    ``prefix_lens[b] + i``; key ``j`` of the request is visible iff
    ``(is_cross_attention or j <= pos) and (W == 0 or j >= pos - W + 1)``.
    Returns ``(total_q, n_q, d)`` in the dtype of ``q``; rows of a request beyond
    ``max_len_extend`` are not computed.  ``validate=True`` (or ``MSGL_DEBUG_CHECKS=1``) first
    checks both offset arrays and that every entry of ``kv_indices`` names a slot of the pool
    (one host synchronisation).
    """
    op = "paged_prefill_attention"
    if q.dim() != 3:
        _fail(op, "q must be 3D (total_q_tokens, num_q_heads, head_dim)")
    if k_cache.dim() != 3 or v_cache.dim() != 3:
        _fail(op, "k_cache and v_cache must be 3D (num_pages, num_kv_heads, head_dim)")
    if (qo_indptr.dim() != 1 or kv_indptr.dim() != 1 or kv_indices.dim() != 1
            or prefix_lens.dim() != 1):
        _fail(op, "qo_indptr, kv_indptr, kv_indices, prefix_lens must be 1D")
    total_q, num_q_heads, head_dim = q.shape
    num_kv_heads = k_cache.shape[1]
    if head_dim not in (128, 256):
        _fail(op, "head_dim must be 128 or 256")
    if num_q_heads % num_kv_heads != 0:
        _fail(op, "num_q_heads must be a multiple of num_kv_heads")
    if k_cache.shape[2] != head_dim or v_cache.shape[2] != head_dim:
        _fail(op, "cache head_dim must match q head_dim")
    if sliding_window_size < 0:
        _fail(op, "sliding_window_size must be >= 0")
    batch = qo_indptr.shape[0] - 1
    if batch <= 0:
        _fail(op, "batch must be > 0")
    if v_cache.shape[1] != num_kv_heads:
        _fail(op, "v_cache shape must match k_cache")
    dtype = _attention_dtype(op, q, k_cache, v_cache, half_ok=False)
    qo_indptr = _int32_1d(op, qo_indptr, "qo_indptr")
    kv_indptr = _int32_1d(op, kv_indptr, "kv_indptr")
    kv_indices = _int32_1d(op, kv_indices, "kv_indices")
    prefix_lens = _int32_1d(op, prefix_lens, "prefix_lens")
    if kv_indptr.shape[0] != batch + 1 or prefix_lens.shape[0] != batch:
        _fail(op, "kv_indptr / prefix_lens length must match qo_indptr")
    dev = _require_device(op, q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices, prefix_lens)
    lib = _lib.load()
    total_kv = kv_indices.shape[0]
    if total_q > 0 and _checks_on(validate):
        _validate_indptr(op, "qo_indptr", qo_indptr, total_q, "q")
        _validate_indptr(op, "kv_indptr", kv_indptr, total_kv, "kv_indices")
        _validate_slot_ids(op, "kv_indices", kv_indices, k_cache.shape[0])
    with _on_device(dev, stream):
        q = q if q.is_contiguous() else q.contiguous()
        out = torch.empty((total_q, num_q_heads, head_dim), dtype=q.dtype, device=dev)
        if total_q == 0:
            return out
        ws_bytes = lib.msgl_paged_prefill_workspace_bytes(
            batch, total_q, total_kv, num_q_heads, num_kv_heads, head_dim, int(max_len_extend))
        ws = _workspace(ws_bytes, dev)
        rc = lib.msgl_paged_prefill_attention(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), qo_indptr.data_ptr(),
            kv_indptr.data_ptr(), kv_indices.data_ptr(), prefix_lens.data_ptr(), out.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws_bytes, batch, total_q, total_kv,
            num_q_heads, num_kv_heads, head_dim, k_cache.shape[0],
            _pool_stride0(op, k_cache, "k_cache"), _pool_stride0(op, v_cache, "v_cache"),
            float(sm_scale), int(max_len_extend), int(bool(is_cross_attention)),
            int(sliding_window_size), dtype, _stream_ptr(stream, dev))
    _check_rc(op, rc)
    return out


def build_attention_metadata(page_table: torch.Tensor, table_rows: torch.Tensor,
                             kv_lens: torch.Tensor, extend_lens: Optional[torch.Tensor] = None, *,
                             total_kv: int, total_q: Optional[int] = None,
                             max_kv_splits: int = 32, stream=None) -> dict:
    """CSR metadata of one step from the slot table, in one launch on the device.

    Device counterpart of ``AttnBackend.build_prefill_metadata`` / ``build_decode_metadata``
    (mini_sglang_mlx/attention/backend.py:205-307), which slice the table per request in
    Python.  ``page_table`` is the ``(rows, max_seq_len)`` int32 slot table, ``table_rows`` /
    ``kv_lens`` / ``extend_lens`` are int32 ``[batch]`` device tensors; ``extend_lens=None``
    builds decode metadata (one query per request).  ``total_kv`` / ``total_q`` are the sums
    of the lengths, which the scheduler knows on the host; they size the outputs.  Returns a
    dict with ``kv_indptr``, ``kv_indices``, ``qo_indptr``, ``prefix_lens``, ``positions``,
    ``num_kv_splits``.
    """
    op = "build_attention_metadata"
    if page_table.dim() != 2:
        _fail(op, "page_table must be 2D (rows, max_seq_len)")
    if page_table.dtype != torch.int32:
        _fail(op, "page_table must be int32")
    if page_table.stride(1) != 1:
        _fail(op, "page_table must be contiguous in its last dimension")
    tensors = [page_table, table_rows, kv_lens] + ([extend_lens] if extend_lens is not None else [])
    for t, name in zip(tensors[1:], ("table_rows", "kv_lens", "extend_lens")):
        if t.dim() != 1:
            _fail(op, f"{name} must be 1D")
    dev = _require_device(op, *tensors)
    table_rows = _int32_1d(op, table_rows, "table_rows")
    kv_lens = _int32_1d(op, kv_lens, "kv_lens")
    batch = kv_lens.shape[0]
    if table_rows.shape[0] != batch:
        _fail(op, "table_rows and kv_lens must have the same length")
    if extend_lens is not None:
        extend_lens = _int32_1d(op, extend_lens, "extend_lens")
        if extend_lens.shape[0] != batch:
            _fail(op, "extend_lens and kv_lens must have the same length")
    if total_q is None:
        total_q = batch if extend_lens is None else 0
    if total_kv < 0 or total_q < 0:
        _fail(op, "total_kv and total_q must be >= 0")
    # one allocation, six views (an allocation per array costs more host time than the kernel)
    sizes = (("kv_indptr", batch + 1), ("qo_indptr", batch + 1), ("prefix_lens", batch),
             ("num_kv_splits", batch), ("positions", total_q), ("kv_indices", total_kv))
    rows = page_table.shape[0]
    stride0 = page_table.stride(0) if rows > 1 else page_table.shape[1]
    with _on_device(dev, stream):
        buf = torch.empty(sum(n for _, n in sizes), dtype=torch.int32, device=dev)
        out, at = {}, 0
        for name, n in sizes:
            out[name] = buf[at:at + n]
            at += n
        rc = _lib.load().msgl_build_attention_metadata(
            page_table.data_ptr(), stride0, rows, page_table.shape[1], table_rows.data_ptr(),
            kv_lens.data_ptr(), extend_lens.data_ptr() if extend_lens is not None else None, batch,
            out["kv_indptr"].data_ptr(), out["kv_indices"].data_ptr(), total_kv,
            out["qo_indptr"].data_ptr(), out["prefix_lens"].data_ptr(), out["positions"].data_ptr(),
            total_q, out["num_kv_splits"].data_ptr(), int(max_kv_splits), _stream_ptr(stream, dev))
    _check_rc(op, rc)
    return out


def _heads_stride0(op: str, t: torch.Tensor, name: str) -> int:
    if t.dim() != 3:
        _fail(op, f"{name} must be 3D (tokens, heads, head_dim)")
    if t.stride(2) != 1 or t.stride(1) != t.shape[2]:
        _fail(op, f"{name} must be contiguous in its (heads, head_dim) dimensions")
    return t.stride(0) if t.shape[0] > 1 else t.shape[1] * t.shape[2]


def qk_norm_rope_store(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_weight: torch.Tensor,
                       k_weight: torch.Tensor, positions: torch.Tensor, out_loc: torch.Tensor,
                       k_cache: torch.Tensor, v_cache: torch.Tensor, *, eps: float,
                       rope_base: float, stream=None,
                       validate: Optional[bool] = None) -> torch.Tensor:
    """Per-head RMSNorm of q and k, rotary embedding of both at ``positions``, and the store of
    the new k and v rows at ``out_loc``, in one pass; returns the rotated q.

    One call for ``q_norm`` / ``k_norm`` / ``rope`` / ``rope`` of the reference's Qwen3 attention
    layer (mini_sglang_mlx/models/qwen3.py:60-68) plus the store that ``AttnBackend.forward``
    does first (attention/backend.py:139).  Attention then runs on the result with no further
    store.  q / k / v may be strided views (tokens, heads, head_dim) of a fused projection.
    """
    op = "qk_norm_rope_store"
    dev = _require_device(op, q, k, v, q_weight, k_weight, positions, out_loc, k_cache, v_cache)
    qs, ks, vs = (_heads_stride0(op, t, n) for t, n in ((q, "q"), (k, "k"), (v, "v")))
    n_tokens, n_q, d = q.shape
    n_kv = k.shape[1]
    if d not in (128, 256):
        _fail(op, "head_dim must be 128 or 256")
    if tuple(k.shape) != (n_tokens, n_kv, d) or tuple(v.shape) != (n_tokens, n_kv, d):
        _fail(op, "k and v shape must be (tokens, num_kv_heads, head_dim)")
    if k_cache.dim() != 3 or tuple(k_cache.shape[1:]) != (n_kv, d) or k_cache.shape != v_cache.shape:
        _fail(op, "k_cache and v_cache must be (num_pages, num_kv_heads, head_dim)")
    for t, name in ((q, "q"), (k, "k"), (v, "v"), (k_cache, "k_cache"), (v_cache, "v_cache"),
                    (q_weight, "q_weight"), (k_weight, "k_weight")):
        if t.dtype != torch.bfloat16:
            _fail(op, f"{name} must be bfloat16")
    if tuple(q_weight.shape) != (d,) or tuple(k_weight.shape) != (d,):
        _fail(op, "q_weight and k_weight must be (head_dim,)")
    positions = _int32_1d(op, positions, "positions")
    out_loc = _int32_1d(op, out_loc, "out_loc")
    if positions.shape[0] != n_tokens or out_loc.shape[0] != n_tokens:
        _fail(op, "positions and out_loc length must match q length")
    if _checks_on(validate):
        _validate_slot_ids(op, "out_loc", out_loc, k_cache.shape[0], unique=True)
    with _on_device(dev, stream):
        q_out = torch.empty((n_tokens, n_q, d), dtype=q.dtype, device=dev)
        q_weight, k_weight = q_weight.contiguous(), k_weight.contiguous()
        rc = _lib.load().msgl_qk_norm_rope_store(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), qs, ks, vs, q_weight.data_ptr(),
            k_weight.data_ptr(), positions.data_ptr(), out_loc.data_ptr(),
            q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
            _pool_stride0(op, k_cache, "k_cache"), _pool_stride0(op, v_cache, "v_cache"),
            k_cache.shape[0], n_tokens, n_q, n_kv, d, float(eps), float(rope_base),
            _lib.MSGL_DTYPE_BF16, _stream_ptr(stream, dev))
    _check_rc(op, rc)
    return q_out


def gdn_state_inplace(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor,
                      beta: torch.Tensor, state: torch.Tensor, slot_ids: torch.Tensor,
                      qo_indptr: torch.Tensor, single_token_mode: bool = False, *,
                      stream=None) -> torch.Tensor:
    """Gated delta-rule recurrence over each request's tokens with the fp32 state of slot
    ``slot_ids[b]`` updated in place; returns ``y`` ``(tokens, hv, dv)`` bf16.

    Drop-in for ``mini_sglang_mlx_kernel.gdn_state_inplace`` (bindings.cpp:56-65,
    gdn_state.cpp:87-135): same argument order, ``single_token_mode`` (decode: one token per
    request, ``qo_indptr`` ignored) and error texts (gdn_state.cpp:26-84, 107-126).
    """
    op = "gdn_state_inplace"
    if q.dim() != 3 or k.dim() != 3:
        _fail(op, "q and k must be 3D")
    if v.dim() != 3:
        _fail(op, "v must be 3D")
    if g.dim() != 2 or beta.dim() != 2:
        _fail(op, "g and beta must be 2D")
    if state.dim() != 4:
        _fail(op, "state must be 4D")
    if slot_ids.dim() != 1 or slot_ids.dtype != torch.int32:
        _fail(op, "slot_ids must be int32 1D")
    if any(t.dtype != torch.bfloat16 for t in (q, k, v, g, beta)):
        _fail(op, "q/k/v/g/beta must be bfloat16")
    if state.dtype != torch.float32:
        _fail(op, "state must be float32")
    if not (q.shape[0] == k.shape[0] == v.shape[0] == g.shape[0] == beta.shape[0]):
        _fail(op, "leading dimensions must match")
    if q.shape[1] != k.shape[1] or q.shape[2] != k.shape[2]:
        _fail(op, "q and k shapes must match")
    if v.shape[1] != g.shape[1] or v.shape[1] != beta.shape[1]:
        _fail(op, "hv dimension mismatch")
    if state.shape[1] != v.shape[1] or state.shape[2] != v.shape[2] or state.shape[3] != q.shape[2]:
        _fail(op, "state shape must be (slots, hv, dv, dk)")
    if v.shape[1] % q.shape[1] != 0:
        _fail(op, "hv must be a multiple of hk")
    if q.shape[2] != 128 or v.shape[2] != 128:
        _fail(op, "this specialized kernel requires dk=dv=128")
    tokens, hk, dk = q.shape
    hv, dv = v.shape[1], v.shape[2]
    batch = slot_ids.shape[0]
    if single_token_mode:
        if tokens != batch:
            _fail(op, "decode mode expects one token per request")
    else:
        if qo_indptr.dim() != 1 or qo_indptr.dtype != torch.int32:
            _fail(op, "qo_indptr must be int32 1D")
        if qo_indptr.shape[0] != batch + 1:
            _fail(op, "qo_indptr must have shape (batch + 1,)")
    dev = _require_device(op, q, k, v, g, beta, state, slot_ids)
    if not single_token_mode and qo_indptr.device != dev:
        _fail(op, "all tensors must be on the same device")
    qs, ks, vs = (_heads_stride0(op, t, n) for t, n in ((q, "q"), (k, "k"), (v, "v")))
    if not (state.stride(3) == 1 and state.stride(2) == dk and state.stride(1) == dv * dk):
        _fail(op, "state must be contiguous in its (hv, dv, dk) dimensions")
    state_stride0 = state.stride(0) if state.shape[0] > 1 else hv * dv * dk
    with _on_device(dev, stream):
        g, beta = g.contiguous(), beta.contiguous()
        slot_ids = slot_ids.contiguous()
        qo_indptr = None if single_token_mode else qo_indptr.contiguous()
        y = torch.empty((tokens, hv, dv), dtype=q.dtype, device=dev)
        rc = _lib.load().msgl_gdn_state_inplace(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), beta.data_ptr(), state.data_ptr(),
            slot_ids.data_ptr(), None if qo_indptr is None else qo_indptr.data_ptr(),
            y.data_ptr(), tokens, batch, hk, hv, dk, dv, state.shape[0], state_stride0, qs, ks, vs,
            1 if single_token_mode else 0, _stream_ptr(stream, dev))
    _check_rc(op, rc)
    return y


def fast_compare_key(a: torch.Tensor, b: torch.Tensor) -> int:
    """Length of the common prefix of two 1-D integer arrays (host tensors).

    Drop-in for ``mini_sglang_mlx_kernel.fast_compare_key`` (fast_compare_key.cpp:9-45): the
    radix tree's key comparison.  Pure host code; device tensors are refused instead of being
    copied behind the caller's back.
    """
    op = "fast_compare_key"
    if a.dim() != 1 or b.dim() != 1:
        _fail(op, "Both arrays must be 1D.")
    if not a.is_contiguous() or not b.is_contiguous():
        _fail(op, "Both arrays must be contiguous.")
    if a.dtype != b.dtype:
        _fail(op, "Both arrays must have the same dtype.")
    if a.dtype not in (torch.int32, torch.int64):
        _fail(op, "Arrays must be int32 or int64.")
    if a.device.type != "cpu" or b.device.type != "cpu":
        _fail(op, "Both arrays must live in host memory.")
    return int(_lib.load().msgl_fast_compare_key(a.data_ptr(), a.numel(), b.data_ptr(), b.numel(),
                                                 a.element_size(), None))
