"""KV-store on the GPU, through the C ABI: bit-exact against the oracle's row scatter."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

SHAPES = [(1, 128, 4, 128), (3, 128, 4, 128), (32, 128, 4, 128), (67, 256, 8, 128),
          (129, 512, 16, 128), (4096, 8192, 8, 128), (5, 64, 1, 256), (7, 33, 3, 36)]


def _bits(t):
    return t.cpu().contiguous().view(torch.int16)


@pytest.mark.parametrize("length,num_pages,n_kv,d", SHAPES)
def test_store_bit_exact(gpu, length, num_pages, n_kv, d):
    from mini_sglang_amd_kernel import store_kv_cache

    print(f"store length={length} pages={num_pages} n_kv={n_kv} d={d}", flush=True)
    g = torch.Generator().manual_seed(1025 + length)
    k = torch.randn((length, n_kv, d), generator=g).to(torch.bfloat16)
    v = torch.randn((length, n_kv, d), generator=g).to(torch.bfloat16)
    kc = torch.randn((num_pages, n_kv, d), generator=g).to(torch.bfloat16)
    vc = torch.randn((num_pages, n_kv, d), generator=g).to(torch.bfloat16)
    loc = torch.randperm(num_pages, generator=g)[:length].to(torch.int32)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    oracle.store_kv_cache(kc_ref, vc_ref, loc, k, v)
    kc_g, vc_g = kc.to(gpu), vc.to(gpu)
    store_kv_cache(kc_g, vc_g, loc.to(gpu), k.to(gpu), v.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(_bits(kc_g), _bits(kc_ref))
    assert torch.equal(_bits(vc_g), _bits(vc_ref))


def test_store_strided_views_and_overwrite(gpu):
    from mini_sglang_amd_kernel import store_kv_cache

    g = torch.Generator().manual_seed(9)
    n_kv, d, n = 2, 128, 11
    kbig = torch.randn((n, 3, n_kv, d), generator=g).to(torch.bfloat16)
    v = torch.randn((n, n_kv, d), generator=g).to(torch.bfloat16)
    kc_big = torch.randn((40, 2, n_kv, d), generator=g).to(torch.bfloat16)
    vc = torch.randn((40, n_kv, d), generator=g).to(torch.bfloat16)
    loc = torch.randperm(40, generator=g)[:n].to(torch.int32)
    kc_ref_big, vc_ref = kc_big.clone(), vc.clone()
    oracle.store_kv_cache(kc_ref_big[:, 1], vc_ref, loc, kbig[:, 2], v)
    kc_g_big, vc_g, kbig_g = kc_big.to(gpu), vc.to(gpu), kbig.to(gpu)
    store_kv_cache(kc_g_big[:, 1], vc_g, loc.to(gpu), kbig_g[:, 2], v.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(_bits(kc_g_big), _bits(kc_ref_big))  # plane 0 untouched, plane 1 written
    assert torch.equal(_bits(vc_g), _bits(vc_ref))
    # overwrite the same slots with other rows (draft calibration pattern)
    oracle.store_kv_cache(kc_ref_big[:, 1], vc_ref, loc, v, kbig[:, 0])
    store_kv_cache(kc_g_big[:, 1], vc_g, loc.to(gpu), v.to(gpu), kbig_g[:, 0])
    torch.cuda.synchronize()
    assert torch.equal(_bits(kc_g_big), _bits(kc_ref_big))
    assert torch.equal(_bits(vc_g), _bits(vc_ref))


def test_store_empty_and_fp32(gpu):
    from mini_sglang_amd_kernel import store_kv_cache

    kc = torch.zeros((4, 2, 8), dtype=torch.float32, device=gpu)
    vc = torch.zeros((4, 2, 8), dtype=torch.float32, device=gpu)
    store_kv_cache(kc, vc, torch.zeros(0, dtype=torch.int32, device=gpu),
                   torch.zeros((0, 2, 8), device=gpu), torch.zeros((0, 2, 8), device=gpu))
    k = torch.arange(32, dtype=torch.float32, device=gpu).reshape(2, 2, 8)
    store_kv_cache(kc, vc, torch.tensor([3, 1], dtype=torch.int32, device=gpu), k, -k)
    torch.cuda.synchronize()
    assert torch.equal(kc[3], k[0]) and torch.equal(vc[1], -k[1])
    assert torch.count_nonzero(kc[0]) == 0 and torch.count_nonzero(kc[2]) == 0
