"""Pools of 4 GiB and more: every byte offset into them needs 64 bits.  Slots are spread over
the whole pool (first and last slot included); the oracle runs on a compacted copy of the
used rows with remapped indices (the result does not depend on where rows live)."""
import math

import pytest
import torch

import oracle
from _util import assert_close_bf16, bf16_randn, indptr

pytestmark = pytest.mark.gpu

N_KV = 8


def _spread_slots(n, num_slots, seed):
    g = torch.Generator().manual_seed(seed)
    s = torch.randperm(num_slots - 2, generator=g)[: n - 2] + 1
    return torch.cat([torch.tensor([num_slots - 1, 0]), s]).to(torch.int32)


@pytest.mark.parametrize("D", [128, 256])
def test_store_decode_and_extend_in_a_pool_over_4gib(gpu, D):
    from mini_sglang_amd_kernel import (paged_decode_attention, paged_prefill_attention,
                                        store_kv_cache)

    NUM_SLOTS = (4 << 30) // (N_KV * D * 2) + 4096  # a little over 4 GiB per pool

    free_b, _ = torch.cuda.mem_get_info()
    if free_b < 12 << 30:
        pytest.skip("needs ~9 GiB of device memory")
    print(f"large pool: {NUM_SLOTS} slots, {NUM_SLOTS * N_KV * D * 2 / 2**30:.2f} GiB each", flush=True)
    kc = torch.empty((NUM_SLOTS, N_KV, D), dtype=torch.bfloat16, device=gpu)
    vc = torch.empty((NUM_SLOTS, N_KV, D), dtype=torch.bfloat16, device=gpu)
    n_q = 32
    kv_lens = [700, 3, 1500]
    ext = [300, 3, 70]           # extend lengths of the prefill call (tile route: 300*4 rows)
    total = sum(kv_lens)
    slots = _spread_slots(total, NUM_SLOTS, 5)
    k_rows = bf16_randn((total, N_KV, D), 11)
    v_rows = bf16_randn((total, N_KV, D), 12)
    # every row goes in through the store kernel
    store_kv_cache(kc, vc, slots.to(gpu), k_rows.to(gpu), v_rows.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(kc[slots.long().to(gpu)].cpu().view(torch.int16), k_rows.view(torch.int16))
    assert torch.equal(vc[-1].cpu().view(torch.int16), v_rows[0].view(torch.int16))

    # compact copy for the oracle: row i of the small pool is slot slots[i]
    small_idx = torch.arange(total, dtype=torch.int32)
    kv_ip = indptr(kv_lens)
    scale = 1.0 / math.sqrt(D)

    # decode over all three requests
    q = bf16_randn((3, n_q, D), 13)
    splits = torch.ones(3, dtype=torch.int32)
    want = oracle.paged_decode_attention(q, k_rows, v_rows, kv_ip, small_idx, splits, scale, 32,
                                         return_f32=True)[1]
    got = paged_decode_attention(q.to(gpu), kc, vc, kv_ip.to(gpu), slots.to(gpu), splits.to(gpu),
                                 scale, 32)
    torch.cuda.synchronize()
    assert_close_bf16(got, want, "decode in a >4 GiB pool")

    # extend (MFMA tile route) and a short verify block (split-K route)
    for name, e in (("extend", ext), ("verify", [4, 3, 4])):
        qq = bf16_randn((sum(e), n_q, D), 14)
        qo_ip = indptr(e)
        prefix = torch.tensor([l - x for l, x in zip(kv_lens, e)], dtype=torch.int32)
        want = oracle.paged_prefill_attention(qq, k_rows, v_rows, qo_ip, kv_ip, small_idx, prefix,
                                              scale, max(e), return_f32=True)[1]
        got = paged_prefill_attention(qq.to(gpu), kc, vc, qo_ip.to(gpu), kv_ip.to(gpu),
                                      slots.to(gpu), prefix.to(gpu), scale, max(e))
        torch.cuda.synchronize()
        assert_close_bf16(got, want, f"{name} in a >4 GiB pool")
    del kc, vc
    torch.cuda.empty_cache()
