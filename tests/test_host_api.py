"""Host-side behaviour that needs no GPU: the C-ABI library loads and exports every symbol
the header declares, argument errors carry the reference's messages
(paged_decode_attention.cpp:25-62, paged_prefill_attention.cpp:31-76, store_kv_cache.cpp:22-63),
metadata builders follow the reference's closed forms (backend.py:205-307), and the product
path refuses to run without a GPU instead of falling back."""
import ctypes
import os
import re
from types import SimpleNamespace

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = sorted(os.path.join(ROOT, "include", f) for f in os.listdir(os.path.join(ROOT, "include"))
                 if f.endswith(".h"))


def _declared_symbols():
    text = "\n".join(open(h).read() for h in HEADERS)
    return sorted(set(re.findall(r"MSGL_API\s+[\w\s\*]+?\b(msgl_\w+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    from mini_sglang_amd_kernel import _lib

    names = _declared_symbols()
    assert names == sorted(_lib.SIGNATURES), "header and ctypes table disagree"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} not exported"
    loaded = _lib.load()
    assert loaded.msgl_version() >= 100
    assert _lib.strerror(0) == "ok"
    assert "head_dim" in _lib.strerror(-2)
    assert _lib.strerror(-9999) == "unknown error code"


def test_c_abi_argument_checks_return_codes_without_touching_a_gpu():
    """Every call below fails validation before any HIP call is made."""
    from mini_sglang_amd_kernel import _lib

    lib = _lib.load()
    fake = ctypes.c_void_p(0x1000)
    # store: head_dim % 4, bad element size, stride smaller than a row
    assert lib.msgl_store_kv_cache(fake, fake, fake, fake, fake, 1, 2, 6, 8, 12, 12, 12, 12, 2, None) == -12
    assert lib.msgl_store_kv_cache(fake, fake, fake, fake, fake, 1, 2, 8, 8, 16, 16, 16, 16, 3, None) == -5
    assert lib.msgl_store_kv_cache(fake, fake, fake, fake, fake, 1, 2, 8, 8, 8, 16, 16, 16, 2, None) == -9
    assert lib.msgl_store_kv_cache(None, fake, fake, fake, fake, 1, 2, 8, 8, 16, 16, 16, 16, 2, None) == -1
    assert lib.msgl_store_kv_cache(None, None, None, None, None, 0, 2, 8, 8, 16, 16, 16, 16, 2, None) == 0
    # decode: head_dim, head ratio, group > 16, dtype, workspace
    def dec(n_q=32, n_kv=8, d=128, dtype=0, ws=fake, ws_bytes=1 << 40, q=fake):
        return lib.msgl_paged_decode_attention(q, fake, fake, fake, fake, fake, fake, ws, ws_bytes,
                                               4, 100, n_q, n_kv, d, 64, n_kv * d, n_kv * d,
                                               0.1, 32, dtype, None)
    assert dec(d=64) == -2
    assert dec(n_q=30) == -3
    assert dec(n_q=34, n_kv=2) == -4
    assert dec(dtype=2) == -5
    assert dec(q=None) == -1
    assert dec(ws=None) == -8
    assert dec(ws_bytes=16) == -8
    # prefill: window, batch
    def pre(batch=2, window=0, d=128, n_q=32, dtype=0):
        return lib.msgl_paged_prefill_attention(fake, fake, fake, fake, fake, fake, fake, fake,
                                                fake, 1 << 40, batch, 16, 100, n_q, 8, d, 64,
                                                8 * d, 8 * d, 0.1, 8, 0, window, dtype, None)
    assert pre(window=-1) == -7
    assert pre(batch=0) == -6
    assert pre(d=96) == -2
    assert pre(n_q=33) == -3
    assert pre(dtype=1) == -5  # float16 exists for decode only
    assert lib.msgl_set_tuning(99, 1) == -9
    assert lib.msgl_paged_decode_workspace_bytes(4, 1000, 32, 8, 128) > 0
    assert lib.msgl_paged_decode_workspace_bytes(4, 1000, 30, 8, 128) == 0
    # prefill workspace: the slots and count words of gang ranges for a launch with several query
    # blocks per (request, kv head) that fills the chip (8 XCDs x 4 gangs x 2 slots x 8 query blocks
    # of 256 rows x 128 floats + 8 waves x 64 lanes x 2 floats; one 8-byte count per (request, kv
    # head, query block)), nothing when they are switched off or at head_dim 256; the partials of a
    # key split for one long request, none again when splitting is switched off
    slot = 256 * 128 * 4 + 8 * 64 * 2 * 4
    assert lib.msgl_paged_prefill_workspace_bytes(8, 4096, 8 * 8704, 32, 8, 128, 512) == 8 * 4 * 2 * 8 * slot + 8 * 8 * 8 * 8
    assert lib.msgl_set_tuning(8, -1) == 0
    assert lib.msgl_paged_prefill_workspace_bytes(8, 4096, 8 * 8704, 32, 8, 128, 512) == 0
    assert lib.msgl_set_tuning(8, 0) == 0
    assert lib.msgl_paged_prefill_workspace_bytes(8, 4096, 8 * 8704, 32, 8, 256, 512) == 0
    one_long = (1, 512, 32768 + 512, 32, 8, 128, 512)
    need = lib.msgl_paged_prefill_workspace_bytes(*one_long)
    assert need > 0 and need % (512 * 32 * (128 + 1) * 4) == 0
    assert lib.msgl_set_tuning(6, 1) == 0
    assert lib.msgl_paged_prefill_workspace_bytes(*one_long) == 0
    assert lib.msgl_set_tuning(6, 0) == 0
    # state pool: size checks come before any pointer is touched; nothing to do is not an error
    def slots(slot_stride=64, row=64, layers=2, num_slots=4, layer_stride=256, pairs=1, slab=fake, dst=fake):
        return lib.msgl_copy_state_slots(slab, layer_stride, slot_stride, row, layers, num_slots, None,
                                         dst, pairs, None)
    assert slots(slot_stride=32) == -9
    assert slots(layer_stride=128) == -9
    assert slots(pairs=-1) == -9
    assert slots(pairs=0) == 0 and slots(layers=0) == 0 and slots(row=0, slot_stride=0, layer_stride=0) == 0
    assert slots(slab=None) == -1 and slots(dst=None) == -1


def _t(shape, dtype=torch.bfloat16):
    return torch.zeros(shape, dtype=dtype)


def _i(n):
    return torch.zeros(n, dtype=torch.int32)


def test_decode_errors_use_the_reference_messages():
    from mini_sglang_amd_kernel import paged_decode_attention as f

    ok = dict(q=_t((2, 16, 128)), k_cache=_t((10, 8, 128)), v_cache=_t((10, 8, 128)),
              kv_indptr=_i(3), kv_indices=_i(5), num_kv_splits=_i(2), sm_scale=0.1, max_kv_splits=32)

    def call(**kw):
        return f(**{**ok, **kw})

    with pytest.raises(RuntimeError, match=r"paged_decode_attention: q must be 3D \(batch, num_q_heads, head_dim\)"):
        call(q=_t((2, 16 * 128)))
    with pytest.raises(RuntimeError, match=r"k_cache and v_cache must be 3D \(num_pages, num_kv_heads, head_dim\)"):
        call(k_cache=_t((10, 8 * 128)))
    with pytest.raises(RuntimeError, match=r"kv_indptr, kv_indices, num_kv_splits must be 1D"):
        call(kv_indptr=torch.zeros((3, 1), dtype=torch.int32))
    with pytest.raises(RuntimeError, match=r"head_dim must be 128 or 256"):
        call(q=_t((2, 16, 64)), k_cache=_t((10, 8, 64)), v_cache=_t((10, 8, 64)))
    with pytest.raises(RuntimeError, match=r"num_q_heads must be a multiple of num_kv_heads"):
        call(q=_t((2, 12, 128)))
    with pytest.raises(RuntimeError, match=r"only q_heads/kv_heads <= 16 is supported"):
        call(q=_t((2, 34, 128)), k_cache=_t((10, 2, 128)), v_cache=_t((10, 2, 128)))
    with pytest.raises(RuntimeError, match=r"cache head_dim must match q head_dim"):
        call(v_cache=_t((10, 8, 256)))
    with pytest.raises(RuntimeError, match=r"unsupported dtype, must be float16 or bfloat16"):
        call(q=_t((2, 16, 128), torch.float32))
    with pytest.raises(RuntimeError, match=r"must be int32"):
        call(kv_indices=torch.zeros(5, dtype=torch.int64))
    # valid arguments on CPU tensors: there is no CPU implementation to fall back to
    with pytest.raises(RuntimeError, match=r"ROCm GPU device"):
        call()


def test_prefill_errors_use_the_reference_messages():
    from mini_sglang_amd_kernel import paged_prefill_attention as f

    ok = dict(q=_t((6, 16, 128)), k_cache=_t((10, 8, 128)), v_cache=_t((10, 8, 128)),
              qo_indptr=_i(3), kv_indptr=_i(3), kv_indices=_i(9), prefix_lens=_i(2),
              sm_scale=0.1, max_len_extend=3)

    def call(**kw):
        return f(**{**ok, **kw})

    with pytest.raises(RuntimeError, match=r"paged_prefill_attention: q must be 3D \(total_q_tokens, num_q_heads, head_dim\)"):
        call(q=_t((6, 2048)))
    with pytest.raises(RuntimeError, match=r"qo_indptr, kv_indptr, kv_indices, prefix_lens must be 1D"):
        call(prefix_lens=torch.zeros((2, 1), dtype=torch.int32))
    with pytest.raises(RuntimeError, match=r"head_dim must be 128 or 256"):
        call(q=_t((6, 16, 96)), k_cache=_t((10, 8, 96)), v_cache=_t((10, 8, 96)))
    with pytest.raises(RuntimeError, match=r"num_q_heads must be a multiple of num_kv_heads"):
        call(q=_t((6, 10, 128)))
    with pytest.raises(RuntimeError, match=r"cache head_dim must match q head_dim"):
        call(k_cache=_t((10, 8, 256)))
    with pytest.raises(RuntimeError, match=r"sliding_window_size must be >= 0"):
        call(sliding_window_size=-1)
    with pytest.raises(RuntimeError, match=r"batch must be > 0"):
        call(qo_indptr=_i(1), kv_indptr=_i(1), prefix_lens=_i(0))
    with pytest.raises(RuntimeError, match=r"ROCm GPU device"):
        call(is_cross_attention=True, sliding_window_size=4)


def test_store_errors_use_the_reference_messages():
    from mini_sglang_amd_kernel import store_kv_cache as f

    ok = dict(k_cache=_t((10, 4, 128)), v_cache=_t((10, 4, 128)), indices=_i(3),
              k=_t((3, 4, 128)), v=_t((3, 4, 128)))

    def call(**kw):
        return f(**{**ok, **kw})

    with pytest.raises(RuntimeError, match=r"store_kv_cache: k_cache and v_cache must be 3D"):
        call(k_cache=_t((10, 512)))
    with pytest.raises(RuntimeError, match=r"indices must be 1D"):
        call(indices=torch.zeros((3, 1), dtype=torch.int32))
    with pytest.raises(RuntimeError, match=r"k and v must be 3D \(length, num_kv_heads, head_dim\)"):
        call(k=_t((3, 512)))
    with pytest.raises(RuntimeError, match=r"k_cache, v_cache, k, v must have the same dtype"):
        call(v=_t((3, 4, 128), torch.float16))
    with pytest.raises(RuntimeError, match=r"indices must be int32"):
        call(indices=torch.zeros(3, dtype=torch.int64))
    with pytest.raises(RuntimeError, match=r"head_dim must be a multiple of 4"):
        call(k_cache=_t((10, 4, 6)), v_cache=_t((10, 4, 6)), k=_t((3, 4, 6)), v=_t((3, 4, 6)))
    with pytest.raises(RuntimeError, match=r"v_cache shape must match k_cache"):
        call(v_cache=_t((11, 4, 128)))
    with pytest.raises(RuntimeError, match=r"k and v shape must be \(length, num_kv_heads, head_dim\)"):
        call(k=_t((4, 4, 128)))
    with pytest.raises(RuntimeError, match=r"ROCm GPU device"):
        call()


def test_mha_kv_cache_and_backend_host_logic():
    from mini_sglang_amd.attention import (MAX_KV_SPLITS, AttnBackend, DecodeMetadata,
                                           PrefillMetadata)
    from mini_sglang_amd.attention.backend import _build_indptr, _compute_num_kv_splits
    from mini_sglang_amd.kvcache import MHAKVCache

    pool = MHAKVCache(num_kv_heads=2, num_layers=3, head_dim=128, num_pages=9,
                      dtype=torch.bfloat16, device="cpu")
    assert pool.num_layers == 3 and pool.dtype == torch.bfloat16
    assert tuple(pool.k_cache(2).shape) == (9, 2, 128)
    assert torch.count_nonzero(pool.v_cache(0)) == 0
    with pytest.raises(AssertionError, match="out_loc must be int32"):
        pool.store_kv(_t((2, 2, 128)), _t((2, 2, 128)), torch.zeros(2, dtype=torch.int64), 0)
    with pytest.raises(ValueError, match="3 slot ids for k of shape"):  # mha_pool.py:42-46
        pool.store_kv(_t((2, 2, 128)), _t((2, 2, 128)), _i(3), 0)
    assert pool.pool_shape == (9, 2, 128) and pool.nbytes == 2 * 3 * 9 * 2 * 128 * 2
    assert pool.k_cache(1).is_contiguous() and pool.k_cache(1).stride(0) == 2 * 128

    # closed forms of backend.py:299-307
    assert _build_indptr([3, 0, 5]).tolist() == [0, 3, 3, 8]
    assert _build_indptr([3, 0, 5]).dtype == torch.int32
    assert _compute_num_kv_splits([1, 128, 129, 4096, 4097, 10**6]).tolist() == [1, 1, 2, 32, 32, 32]
    assert MAX_KV_SPLITS == 32

    page_table = torch.arange(4 * 20, dtype=torch.int32).reshape(4, 20) * 3 % 61
    be = AttnBackend(SimpleNamespace(head_dim=128), pool, page_table)
    assert abs(be.sm_scale - 128 ** -0.5) < 1e-12
    reqs = [SimpleNamespace(table_idx=2, extend_len=3, device_len=7, cached_len=4),
            SimpleNamespace(table_idx=0, extend_len=5, device_len=5, cached_len=0)]
    md = be.build_prefill_metadata(reqs)
    assert isinstance(md, PrefillMetadata)
    assert md.qo_indptr.tolist() == [0, 3, 8] and md.kv_indptr.tolist() == [0, 7, 12]
    assert md.prefix_lens.tolist() == [4, 0] and md.max_len_extend == 5
    assert md.positions.tolist() == [4, 5, 6, 0, 1, 2, 3, 4]
    assert md.kv_indices.tolist() == page_table[2, :7].tolist() + page_table[0, :5].tolist()
    assert md.get_last_indices(2).tolist() == [2, 7]
    # virtual extend window (speculative verify, spec_engine.py:205-212): K+1 = 4 positions
    mv = be.build_prefill_metadata(reqs, extend_lens=[4, 4], kv_lens=[11, 9])
    assert mv.prefix_lens.tolist() == [7, 5] and mv.max_len_extend == 4
    assert mv.positions.tolist() == [7, 8, 9, 10, 5, 6, 7, 8]
    dm = be.build_decode_metadata(reqs)
    assert isinstance(dm, DecodeMetadata)
    assert dm.kv_indptr.tolist() == [0, 7, 12] and dm.positions.tolist() == [4, 0]
    assert dm.num_kv_splits.tolist() == [1, 1] and dm.max_kv_splits == 32
    assert dm.get_last_indices(2).tolist() == [0, 1]
    batch = SimpleNamespace(padded_reqs=reqs, is_prefill=False, attn_metadata=None)
    be.prepare_metadata(batch)
    assert isinstance(batch.attn_metadata, DecodeMetadata)
    # decode rejects the mask flags, forward rejects a negative window (backend.py:134,158-162)
    batch.out_loc = _i(2)
    with pytest.raises(AssertionError, match="sliding_window_size must be >= 0"):
        be.forward(_t((2, 4, 128)), _t((2, 2, 128)), _t((2, 2, 128)), 0, batch, sliding_window_size=-1)


def test_workload_generators_are_consistent():
    from mini_sglang_amd import roofline
    from mini_sglang_amd.workloads import config_workload

    for cfg, variant in [(1, ""), (2, ""), (3, ""), (4, ""), (5, ""), (5, "window")]:
        wl = config_workload(cfg, scale=0.02, variant=variant)
        n_slots = wl.k_cache.shape[0]
        idx = wl.kv_indices.long()
        assert idx.numel() == sum(wl.kv_lens) == int(wl.kv_indptr[-1])
        assert int(idx.min()) >= 0 and int(idx.max()) < n_slots
        assert idx.unique().numel() == idx.numel(), "slots must not be shared between tokens"
        ip = wl.kv_indptr.tolist()
        for b in range(wl.batch):
            s = idx[ip[b]:ip[b + 1]]
            t = torch.arange(s.numel())
            # page-granular layout: slot = page * 16 + t % 16, one page id per 16 tokens
            assert torch.equal(s % wl.page_size, t % wl.page_size)
            pages = s // wl.page_size
            assert torch.equal(pages, pages[(t // wl.page_size) * wl.page_size])
        if wl.out_loc is not None:
            assert wl.out_loc.numel() == sum(wl.extend_lens)
        assert wl.attention_bytes() > 0 and wl.attention_flops() > 0
    # closed forms of the algorithmic work on a case small enough to count by hand
    assert roofline.visible_pairs(prefix=4, q_len=4, kv_len=8, is_cross=False, window=5) == 5 + 5 + 5 + 5
    assert roofline.visible_pairs(prefix=0, q_len=4, kv_len=4, is_cross=False, window=0) == 10
    assert roofline.visible_pairs(prefix=6, q_len=2, kv_len=8, is_cross=True, window=3) == 4 + 3
    assert roofline.visible_range(6, 2, 8, True, 3) == (4, 8)
    assert roofline.decode_bytes([10], 4, 2, 128) == 10 * (2 * 2 * 128 * 2 + 4) + 2 * 4 * 128 * 2


# ---- opt-in index validation in front of the launches (host-forcible: plain tensors) -----------
def test_slot_id_validation_names_range_and_duplicates():
    import mini_sglang_amd_kernel as mk

    ok = torch.tensor([5, 0, 3], dtype=torch.int32)
    mk._validate_slot_ids("store_kv_cache", "indices", ok, 6, unique=True)
    mk._validate_slot_ids("store_kv_cache", "indices", ok[:0], 0, unique=True)  # nothing to check
    for bad in ([1, 6], [-1, 2], [2 ** 31 - 1]):
        with pytest.raises(RuntimeError, match=r"store_kv_cache: indices holds slot ids outside \[0, 6\)"):
            mk._validate_slot_ids("store_kv_cache", "indices", torch.tensor(bad, dtype=torch.int32), 6)
    twice = torch.tensor([4, 2, 4, 2, 1], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="2 duplicate slot id"):
        mk._validate_slot_ids("store_kv_cache", "indices", twice, 6, unique=True)
    mk._validate_slot_ids("paged_decode_attention", "kv_indices", twice, 6)  # readers may repeat


def test_indptr_validation():
    import mini_sglang_amd_kernel as mk

    t = lambda v: torch.tensor(v, dtype=torch.int32)
    mk._validate_indptr("op", "kv_indptr", t([0, 4, 4, 9]), 9, "kv_indices")
    with pytest.raises(RuntimeError, match="non-decreasing"):
        mk._validate_indptr("op", "kv_indptr", t([0, 4, 3]), 9, "kv_indices")
    with pytest.raises(RuntimeError, match="non-decreasing"):
        mk._validate_indptr("op", "kv_indptr", t([-1, 4]), 9, "kv_indices")
    with pytest.raises(RuntimeError, match="ends at 10, beyond the 9 entries of kv_indices"):
        mk._validate_indptr("op", "kv_indptr", t([0, 10]), 9, "kv_indices")


def test_validation_is_off_unless_asked_for(monkeypatch):
    import mini_sglang_amd_kernel as mk

    monkeypatch.delenv("MSGL_DEBUG_CHECKS", raising=False)
    assert mk._checks_on(None) is False and mk._checks_on(False) is False
    assert mk._checks_on(True) is True
    monkeypatch.setenv("MSGL_DEBUG_CHECKS", "1")
    assert mk._checks_on(None) is True
    assert mk._checks_on(False) is False  # the call's own word wins
    monkeypatch.setenv("MSGL_DEBUG_CHECKS", "0")
    assert mk._checks_on(None) is False


def test_tuning_knobs_are_per_host_thread():
    """msgl_set_tuning acts on the calling thread only; msgl_get_tuning shows what a thread's own
    launches and workspace queries use."""
    import threading

    from mini_sglang_amd_kernel import _lib

    lib = _lib.load()
    cfg3 = (8, 4096, 8 * 8704, 32, 8, 128, 512)
    with_gangs = lib.msgl_paged_prefill_workspace_bytes(*cfg3)
    assert with_gangs > 0
    _lib.set_tuning(_lib.TUNE_PREFILL_GANGS, -1)
    try:
        assert _lib.get_tuning(_lib.TUNE_PREFILL_GANGS) == -1
        assert lib.msgl_paged_prefill_workspace_bytes(*cfg3) == 0
        seen = {}

        def other():
            seen["knob"] = _lib.get_tuning(_lib.TUNE_PREFILL_GANGS)
            seen["bytes"] = lib.msgl_paged_prefill_workspace_bytes(*cfg3)
            _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, 3)
            seen["own"] = _lib.get_tuning(_lib.TUNE_PREFILL_KEY_SPLITS)

        t = threading.Thread(target=other)
        t.start()
        t.join()
        assert seen == {"knob": 0, "bytes": with_gangs, "own": 3}
        assert _lib.get_tuning(_lib.TUNE_PREFILL_KEY_SPLITS) == 0  # the other thread's value stayed there
    finally:
        _lib.set_tuning(_lib.TUNE_PREFILL_GANGS, 0)
    assert _lib.get_tuning(_lib.TUNE_PREFILL_GANGS) == 0
    out = __import__("ctypes").c_int64(5)
    assert lib.msgl_get_tuning(99, __import__("ctypes").byref(out)) == -9
    assert lib.msgl_get_tuning(0, None) == -1
