"""Run a workload through the HIP operators (C ABI) and through the CPU oracle."""
from __future__ import annotations

import torch

import oracle


def run_gpu(wl, device, store=True):
    """Returns (out_cpu, k_cache_cpu, v_cache_cpu) after the GPU path."""
    from mini_sglang_amd_kernel import (paged_decode_attention, paged_prefill_attention,
                                        store_kv_cache)

    g = wl.to(device)
    if store and g.out_loc is not None:
        store_kv_cache(g.k_cache, g.v_cache, g.out_loc, g.new_k, g.new_v)
    if g.kind == "decode":
        out = paged_decode_attention(g.q, g.k_cache, g.v_cache, g.kv_indptr, g.kv_indices,
                                     g.num_kv_splits, g.sm_scale, g.max_kv_splits)
    else:
        out = paged_prefill_attention(
            g.q, g.k_cache, g.v_cache, g.qo_indptr, g.kv_indptr, g.kv_indices, g.prefix_lens,
            g.sm_scale, g.max_len_extend, is_cross_attention=g.is_cross_attention,
            sliding_window_size=g.sliding_window_size)
    torch.cuda.synchronize()
    return out.cpu(), g


def run_oracle(wl, store=True, precision="f64"):
    """Returns the oracle's fp32 output; stores into copies of the pools first."""
    c = wl.clone_pools() if (store and wl.out_loc is not None) else wl
    if store and c.out_loc is not None:
        oracle.store_kv_cache(c.k_cache, c.v_cache, c.out_loc, c.new_k, c.new_v)
    if c.kind == "decode":
        out = oracle.paged_decode_attention(c.q, c.k_cache, c.v_cache, c.kv_indptr, c.kv_indices,
                                            c.num_kv_splits, c.sm_scale, c.max_kv_splits,
                                            precision=precision, return_f32=True)[1]
    else:
        out = oracle.paged_prefill_attention(
            c.q, c.k_cache, c.v_cache, c.qo_indptr, c.kv_indptr, c.kv_indices, c.prefix_lens,
            c.sm_scale, c.max_len_extend, is_cross_attention=c.is_cross_attention,
            sliding_window_size=c.sliding_window_size, precision=precision, return_f32=True)[1]
    return out, c
