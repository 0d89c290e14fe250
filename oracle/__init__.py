"""CPU oracle for the paged-attention path -- TEST INFRASTRUCTURE, not product code.

Thin ctypes front end over ``paged_attention_oracle.c`` (built by ``oracle/Makefile``).
Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this package; the product path never does.

Every function takes CPU ``torch`` tensors with the reference operator's argument
order and meaning (mini-sglang-mlx-kernel/csrc/bindings.cpp:27-55) and returns CPU
tensors.  ``precision="f64"`` (default) is the checker; ``precision="f32"`` is the
OpenMP float build that bench.py times as the CPU baseline.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Tuple

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIBS = {}

_i64 = ctypes.c_int64
_i32 = ctypes.c_int32
_f32 = ctypes.c_float
_vp = ctypes.c_void_p


def build(force: bool = False) -> None:
    """Compile both oracle variants with gcc (``make -C oracle``)."""
    args = ["make", "-C", _HERE]
    if force:
        args.insert(1, "-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)
    _LIBS.clear()


def _lib(precision: str) -> ctypes.CDLL:
    if precision not in ("f64", "f32"):
        raise ValueError(f"precision must be 'f64' or 'f32', got {precision!r}")
    lib = _LIBS.get(precision)
    if lib is not None:
        return lib
    path = os.path.join(_HERE, f"liboracle_{precision}.so")
    if not os.path.exists(path):
        build()
    lib = ctypes.CDLL(path)
    lib.oracle_acc_bytes.restype = ctypes.c_int
    lib.oracle_store_kv_cache.restype = None
    lib.oracle_store_kv_cache.argtypes = [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                          _i64, _i64, _i32]
    lib.oracle_paged_prefill_attention.restype = None
    lib.oracle_paged_prefill_attention.argtypes = [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
        _f32, _i64, _i32, _i64]
    lib.oracle_paged_decode_attention.restype = None
    lib.oracle_paged_decode_attention.argtypes = [
        _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
        _i64, _f32, _i64]
    lib.oracle_decode_kv_len_per_split.restype = _i64
    lib.oracle_decode_kv_len_per_split.argtypes = [_i64, _i64]
    lib.oracle_f32_to_bf16.restype = None
    lib.oracle_f32_to_bf16.argtypes = [_vp, _vp, _i64]
    lib.oracle_bf16_to_f32.restype = None
    lib.oracle_bf16_to_f32.argtypes = [_vp, _vp, _i64]
    assert lib.oracle_acc_bytes() == (8 if precision == "f64" else 4)
    _LIBS[precision] = lib
    return lib


def _cpu(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.device.type != "cpu":
        raise ValueError(f"oracle: {name} must be a CPU tensor")
    return t


def _bits(t: torch.Tensor, name: str) -> torch.Tensor:
    """bf16 tensor -> same memory viewed as int16 (bit patterns)."""
    _cpu(t, name)
    if t.dtype != torch.bfloat16:
        raise ValueError(f"oracle: {name} must be bfloat16, got {t.dtype}")
    return t.view(torch.int16)


def _idx(t: torch.Tensor, name: str) -> torch.Tensor:
    _cpu(t, name)
    if t.dtype != torch.int32:
        raise ValueError(f"oracle: {name} must be int32")
    return t.contiguous()


def _pool_stride(pool: torch.Tensor, name: str) -> int:
    if pool.dim() != 3 or pool.stride(2) != 1 or pool.stride(1) != pool.shape[2]:
        raise ValueError(f"oracle: {name} must be (slots, n_kv, d) with contiguous inner dims")
    return pool.stride(0)


def store_kv_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, indices: torch.Tensor,
                   k: torch.Tensor, v: torch.Tensor) -> None:
    """In place ``k_cache[indices[r]] = k[r]``, ``v_cache[indices[r]] = v[r]`` (bit copy)."""
    lib = _lib("f64")
    for t, n in ((k_cache, "k_cache"), (v_cache, "v_cache"), (k, "k"), (v, "v")):
        _cpu(t, n)
        if t.dim() != 3 or t.stride(2) != 1 or t.stride(1) != t.shape[2]:
            raise ValueError(f"oracle: {n} must be 3-D with contiguous inner dims")
    indices = _idx(indices, "indices")
    row = k_cache.shape[1] * k_cache.shape[2]
    lib.oracle_store_kv_cache(
        k_cache.data_ptr(), v_cache.data_ptr(), indices.data_ptr(), k.data_ptr(),
        v.data_ptr(), indices.numel(), row, k_cache.stride(0), v_cache.stride(0),
        k.stride(0), v.stride(0), k_cache.element_size())


def paged_prefill_attention(q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices,
                            prefix_lens, sm_scale: float, max_len_extend: int, *,
                            is_cross_attention: bool = False, sliding_window_size: int = 0,
                            precision: str = "f64",
                            return_f32: bool = False):
    """Extend attention; returns bf16 ``(total_q, n_q, d)`` (and the unrounded fp32)."""
    lib = _lib(precision)
    qb = _bits(q.contiguous(), "q")
    kb, vb = _bits(k_cache, "k_cache"), _bits(v_cache, "v_cache")
    ks, vs = _pool_stride(k_cache, "k_cache"), _pool_stride(v_cache, "v_cache")
    qo_indptr, kv_indptr = _idx(qo_indptr, "qo_indptr"), _idx(kv_indptr, "kv_indptr")
    kv_indices, prefix_lens = _idx(kv_indices, "kv_indices"), _idx(prefix_lens, "prefix_lens")
    total_q, n_q, d = q.shape
    n_kv = k_cache.shape[1]
    out_f32 = torch.zeros((total_q, n_q, d), dtype=torch.float32)
    out_bf16 = torch.zeros((total_q, n_q, d), dtype=torch.bfloat16)
    lib.oracle_paged_prefill_attention(
        qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), qo_indptr.data_ptr(),
        kv_indptr.data_ptr(), kv_indices.data_ptr(), prefix_lens.data_ptr(),
        out_f32.data_ptr(), out_bf16.data_ptr(), qo_indptr.numel() - 1, n_q, n_kv, d, ks,
        vs, float(sm_scale), int(max_len_extend), int(bool(is_cross_attention)),
        int(sliding_window_size))
    return (out_bf16, out_f32) if return_f32 else out_bf16


def paged_decode_attention(q, k_cache, v_cache, kv_indptr, kv_indices, num_kv_splits,
                           sm_scale: float, max_kv_splits: int, *, precision: str = "f64",
                           return_f32: bool = False, return_partials: bool = False):
    """Split-K decode as the reference stages it; returns bf16 ``(batch, n_q, d)``.

    ``return_partials`` adds ``(att_out, att_lse)``, the stage-1 buffers of
    paged_decode_attention.cpp:118-129 (entries of empty splits are left at zero).
    """
    lib = _lib(precision)
    qb = _bits(q.contiguous(), "q")
    kb, vb = _bits(k_cache, "k_cache"), _bits(v_cache, "v_cache")
    ks, vs = _pool_stride(k_cache, "k_cache"), _pool_stride(v_cache, "v_cache")
    kv_indptr, kv_indices = _idx(kv_indptr, "kv_indptr"), _idx(kv_indices, "kv_indices")
    num_kv_splits = _idx(num_kv_splits, "num_kv_splits")
    batch, n_q, d = q.shape
    n_kv = k_cache.shape[1]
    out_f32 = torch.zeros((batch, n_q, d), dtype=torch.float32)
    out_bf16 = torch.zeros((batch, n_q, d), dtype=torch.bfloat16)
    att_out = torch.zeros((batch, n_q, max_kv_splits, d), dtype=torch.float32)
    att_lse = torch.zeros((batch, n_q, max_kv_splits), dtype=torch.float32)
    lib.oracle_paged_decode_attention(
        qb.data_ptr(), kb.data_ptr(), vb.data_ptr(), kv_indptr.data_ptr(),
        kv_indices.data_ptr(), num_kv_splits.data_ptr(), out_f32.data_ptr(),
        out_bf16.data_ptr(), att_out.data_ptr(), att_lse.data_ptr(), batch, n_q, n_kv, d,
        ks, vs, float(sm_scale), int(max_kv_splits))
    res = [out_bf16]
    if return_f32:
        res.append(out_f32)
    if return_partials:
        res += [att_out, att_lse]
    return res[0] if len(res) == 1 else tuple(res)


def decode_kv_len_per_split(seq_len: int, kv_splits: int) -> int:
    """Split length of paged_decode_attention.metal:356-360."""
    return int(_lib("f64").oracle_decode_kv_len_per_split(int(seq_len), int(kv_splits)))


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    _lib("f64").oracle_f32_to_bf16(x.ctypes.data, out.ctypes.data, x.size)
    return out


def bf16_bits_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    _lib("f64").oracle_bf16_to_f32(x.ctypes.data, out.ctypes.data, x.size)
    return out
