"""The decode entry point that allocates nothing (msgl_paged_decode_attention_noalloc): same bits
as msgl_paged_decode_attention, through the C ABI, on two calls in a row that share the library's
built-in scratch array, the second with a smaller input; sizes beyond the array are refused before
anything is launched."""
import pytest
import torch

from mini_sglang_amd.workloads import build_workload

pytestmark = pytest.mark.gpu


def _call(lib, g, entry, out, ws=None):
    batch, n_q, d = g.q.shape
    total_kv = g.kv_indices.shape[0]
    head = [g.q.data_ptr(), g.k_cache.data_ptr(), g.v_cache.data_ptr(), g.kv_indptr.data_ptr(),
            g.kv_indices.data_ptr(), g.num_kv_splits.data_ptr(), out.data_ptr()]
    tail = [batch, total_kv, n_q, g.k_cache.shape[1], d, g.k_cache.shape[0], g.k_cache.stride(0),
            g.v_cache.stride(0), float(g.sm_scale), int(g.max_kv_splits), 0, None]
    if entry == "noalloc":
        return lib.msgl_paged_decode_attention_noalloc(*head, *tail)
    return lib.msgl_paged_decode_attention(*head, ws.data_ptr(), ws.numel(), *tail)


def _both(lib, wl, gpu, what):
    g = wl.to(gpu)
    batch, n_q, d = g.q.shape
    ws_bytes = lib.msgl_paged_decode_workspace_bytes(batch, g.kv_indices.shape[0], n_q,
                                                     g.k_cache.shape[1], d)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=gpu)
    want = torch.full_like(g.q, 3.0)
    got = torch.full_like(g.q, 5.0)
    print(f"no-alloc decode, {what}: batch {batch}, {g.kv_indices.shape[0]} kv tokens, "
          f"{ws_bytes} workspace bytes", flush=True)
    assert _call(lib, g, "workspace", want, ws) == 0
    assert _call(lib, g, "noalloc", got) == 0
    torch.cuda.synchronize()
    assert torch.equal(got.cpu().view(torch.int16), want.cpu().view(torch.int16)), what
    return g


def test_noalloc_decode_equals_the_workspace_entry_point_twice_in_a_row(gpu):
    from mini_sglang_amd_kernel import _lib

    lib = _lib.load()
    # first call: requests cut over many segments (partials of every request in the scratch)
    big = build_workload("t", "decode", seed=21, n_q=32, n_kv=8,
                         kv_lens=[4096, 1500, 9000, 33, 0, 2049, 7000, 640], pool_factor=1.2)
    _both(lib, big, gpu, "first call")
    # second call, smaller, straight after: what the first call left in the scratch must not leak
    small = build_workload("t", "decode", seed=22, n_q=32, n_kv=8, kv_lens=[700, 5, 1300],
                           pool_factor=1.2)
    _both(lib, small, gpu, "second call, smaller")
    _both(lib, big, gpu, "third call, the first shape again")


def test_noalloc_decode_other_head_shapes(gpu):
    from mini_sglang_amd_kernel import _lib

    lib = _lib.load()
    for n_q, n_kv, d in ((16, 8, 128), (64, 8, 128), (8, 1, 128), (16, 4, 256)):
        wl = build_workload("t", "decode", seed=23 + n_q, n_q=n_q, n_kv=n_kv, head_dim=d,
                            kv_lens=[3000, 17, 1024, 5000], pool_factor=1.1)
        _both(lib, wl, gpu, f"heads {n_q}/{n_kv} head_dim {d}")


def test_noalloc_decode_refuses_sizes_beyond_its_scratch(gpu):
    from mini_sglang_amd_kernel import _lib

    lib = _lib.load()
    # 4096 requests: (segments + batch) * n_q * (d + 1) * 4 bytes is far beyond 8 MiB
    wl = build_workload("t", "decode", seed=29, n_q=32, n_kv=8, kv_lens=[16] * 4096, pool_factor=1.0)
    g = wl.to(gpu)
    need = lib.msgl_paged_decode_workspace_bytes(4096, g.kv_indices.shape[0], 32, 8, 128)
    assert need > 8 * 1024 * 1024
    out = torch.full_like(g.q, 5.0)
    print("no-alloc decode: over the scratch limit", flush=True)
    rc = _call(lib, g, "noalloc", out)
    assert rc == -14 and "scratch" in _lib.strerror(rc)
    torch.cuda.synchronize()
    assert (out.float() == 5.0).all()  # nothing was launched
