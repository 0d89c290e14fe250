"""``AttnBackend.store_kv_only``: the draft-calibration pattern of the reference
(mini_sglang_mlx/attention/backend.py:174-196, caller models/dflash.py:259-261).

A proposal forward writes K/V rows for a verify-shaped block (a few new tokens per request on a
cached prefix) and attends; calibration then overwrites the SAME slots with other rows through
``store_kv_only``; attention issued afterwards must see the new rows.  Both attention results are
checked against the oracle on pools the oracle stored into itself, and the GPU pools must equal
those pools bit for bit after each store.  Every mask the draft layers use is covered
(models/dflash.py:300-304: causal, full, and their windowed forms)."""
import pytest
import torch

import oracle
from _util import assert_close_bf16, bf16_randn, indptr
from test_oracle_metadata import _Req

pytestmark = pytest.mark.gpu

N_Q, N_KV, D = 32, 8, 128
K_PLUS_1 = 8  # tokens per request in one verify / proposal block


class _Cfg:
    head_dim = D


class _Batch:
    pass


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16)


@pytest.mark.parametrize("is_cross,window", [(False, 0), (True, 0), (False, 48), (True, 48)],
                         ids=["causal", "full", "causal_window", "bidirectional_window"])
@pytest.mark.parametrize("extend", [K_PLUS_1, 96], ids=["verify_block", "tile_kernel_block"])
def test_overwrite_through_store_kv_only_is_what_attention_then_reads(gpu, is_cross, window, extend):
    from mini_sglang_amd.attention.backend import AttnBackend
    from mini_sglang_amd.kvcache import MHAKVCache

    prefixes = [200, 37, 1000, 0]
    batch = len(prefixes)
    slots, max_seq = 4096, 1200
    g = torch.Generator().manual_seed(77 + extend + window)
    perm = torch.randperm(slots - 1, generator=g).to(torch.int32)  # last slot = the dummy slot
    table = torch.zeros((batch + 1, max_seq), dtype=torch.int32)
    at = 0
    for b, p in enumerate(prefixes):
        table[b, : p + extend] = perm[at : at + p + extend]
        at += p + extend

    kv = MHAKVCache(num_kv_heads=N_KV, num_layers=2, head_dim=D, num_pages=slots,
                    dtype=torch.bfloat16, device=gpu)
    layer = 1
    # the cached prefixes: random rows everywhere (also in slots nobody references)
    kv.k_cache(layer).copy_(bf16_randn((slots, N_KV, D), 1).to(gpu))
    kv.v_cache(layer).copy_(bf16_randn((slots, N_KV, D), 2).to(gpu))
    ref_k, ref_v = kv.k_cache(layer).cpu().clone(), kv.v_cache(layer).cpu().clone()
    backend = AttnBackend(_Cfg(), kv, table.to(gpu))

    reqs = [_Req(b, p, p + extend) for b, p in enumerate(prefixes)]
    bt = _Batch()
    bt.attn_metadata = backend.build_prefill_metadata(reqs)
    out_loc = torch.cat([table[b, p : p + extend] for b, p in enumerate(prefixes)])
    bt.out_loc = out_loc.to(gpu)
    total = batch * extend
    q = bf16_randn((total, N_Q, D), 3)
    qo, kvp = indptr([extend] * batch), indptr([p + extend for p in prefixes])
    kv_indices = torch.cat([table[b, : p + extend] for b, p in enumerate(prefixes)])
    prefix_lens = torch.tensor(prefixes, dtype=torch.int32)

    def oracle_attend():
        return oracle.paged_prefill_attention(
            q, ref_k, ref_v, qo, kvp, kv_indices, prefix_lens, D ** -0.5, extend,
            is_cross_attention=is_cross, sliding_window_size=window, precision="f64",
            return_f32=True)[1]

    what = f"cross={is_cross} W={window} extend={extend}"
    # 1. proposal forward: store, then attend
    k1, v1 = bf16_randn((total, N_KV, D), 4), bf16_randn((total, N_KV, D), 5)
    print(f"store_kv_only {what}: proposal forward", flush=True)
    got1 = backend.forward(q.to(gpu), k1.to(gpu), v1.to(gpu), layer, bt,
                           is_cross_attention=is_cross, sliding_window_size=window)
    torch.cuda.synchronize()
    oracle.store_kv_cache(ref_k, ref_v, out_loc, k1, v1)
    assert torch.equal(_bits(kv.k_cache(layer)), _bits(ref_k)), what
    assert torch.equal(_bits(kv.v_cache(layer)), _bits(ref_v)), what
    assert_close_bf16(got1, oracle_attend(), f"{what}: proposal forward")

    # 2. calibration: other rows into the same slots, no attention
    k2, v2 = bf16_randn((total, N_KV, D), 6), bf16_randn((total, N_KV, D), 7)
    print(f"store_kv_only {what}: overwrite", flush=True)
    assert backend.store_kv_only(k2.to(gpu), v2.to(gpu), bt.out_loc, layer) is None
    torch.cuda.synchronize()
    oracle.store_kv_cache(ref_k, ref_v, out_loc, k2, v2)
    assert torch.equal(_bits(kv.k_cache(layer)), _bits(ref_k)), what
    assert torch.equal(_bits(kv.v_cache(layer)), _bits(ref_v)), what
    # the other layer's pools were never touched
    assert not kv.k_cache(0).any() and not kv.v_cache(0).any()

    # 3. attention on the calibrated pool (no store): sees the new rows, not the old ones
    print(f"store_kv_only {what}: attend again", flush=True)
    got2 = backend._attend(q.to(gpu), kv.k_cache(layer), kv.v_cache(layer), bt.attn_metadata,
                           is_cross, window)
    torch.cuda.synchronize()
    assert_close_bf16(got2, oracle_attend(), f"{what}: after calibration")
    assert (got2.float() - got1.float()).abs().max() > 0.05, "the overwrite changed nothing"


def test_store_kv_only_checks_lengths_like_the_pool(gpu):
    """The reference raises ValueError on a length mismatch (kvcache/mha_pool.py:42-46) and
    asserts int32 slot ids (:38); store_kv_only goes through the same pool method."""
    from mini_sglang_amd.attention.backend import AttnBackend
    from mini_sglang_amd.kvcache import MHAKVCache

    kv = MHAKVCache(num_kv_heads=2, num_layers=1, head_dim=D, num_pages=64,
                    dtype=torch.bfloat16, device=gpu)
    backend = AttnBackend(_Cfg(), kv, torch.zeros((2, 8), dtype=torch.int32, device=gpu))
    k = torch.zeros((3, 2, D), dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError):
        backend.store_kv_only(k, k, torch.zeros(4, dtype=torch.int32, device=gpu), 0)
    with pytest.raises(AssertionError):
        backend.store_kv_only(k, k, torch.zeros(3, dtype=torch.int64, device=gpu), 0)
