"""Index validation switched on with valid inputs (results must not change), and the writer
kernels' own guard: a slot id outside the pool stores nothing.  The error paths of the validation
itself are host tests (tests/test_host_api.py); no test here hands a reader kernel a bad index."""
import pytest
import torch

from _gpu_util import run_gpu
from _util import bf16_randn
from mini_sglang_amd.workloads import build_workload

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16)


@pytest.mark.parametrize("kind", ["decode", "verify", "extend"])
def test_valid_inputs_pass_validation_and_give_the_same_bits(gpu, kind, monkeypatch):
    if kind == "decode":
        wl = build_workload("t", "decode", seed=11, n_q=16, n_kv=4, kv_lens=[70, 1, 0, 900])
    else:
        ext = [8, 8, 5] if kind == "verify" else [130, 64, 200]
        wl = build_workload("t", "prefill", seed=12, n_q=16, n_kv=4,
                            kv_lens=[300 + ext[0], ext[1], 1000 + ext[2]], extend_lens=ext,
                            store_new=True)
    print(f"validation on, {kind}", flush=True)
    monkeypatch.delenv("MSGL_DEBUG_CHECKS", raising=False)
    plain, g0 = run_gpu(wl, gpu)
    monkeypatch.setenv("MSGL_DEBUG_CHECKS", "1")
    checked, g1 = run_gpu(wl, gpu)
    assert torch.equal(_bits(plain), _bits(checked))
    assert torch.equal(_bits(g0.k_cache), _bits(g1.k_cache))


def test_validation_rejects_before_any_launch(gpu):
    """The check runs on the device and raises on the host; the pools are untouched."""
    from mini_sglang_amd_kernel import store_kv_cache

    kc = torch.zeros((32, 2, 128), dtype=torch.bfloat16, device=gpu)
    vc = torch.zeros_like(kc)
    k = bf16_randn((3, 2, 128), 1).to(gpu)
    print("validation: duplicate and out-of-range store indices", flush=True)
    with pytest.raises(RuntimeError, match="duplicate slot id"):
        store_kv_cache(kc, vc, torch.tensor([4, 9, 4], dtype=torch.int32, device=gpu), k, k, validate=True)
    with pytest.raises(RuntimeError, match=r"outside \[0, 32\)"):
        store_kv_cache(kc, vc, torch.tensor([4, 32, 5], dtype=torch.int32, device=gpu), k, k, validate=True)
    torch.cuda.synchronize()
    assert not kc.any() and not vc.any()


def test_store_skips_rows_whose_slot_is_outside_the_pool(gpu):
    """Defined behaviour of the two writer kernels: such a row is dropped, the others land."""
    from mini_sglang_amd_kernel import qk_norm_rope_store, store_kv_cache

    slots, n_kv, d = 40, 4, 128
    kc = torch.zeros((slots + 8, n_kv, d), dtype=torch.bfloat16, device=gpu)  # 8 guard rows
    vc = torch.zeros_like(kc)
    k, v = bf16_randn((5, n_kv, d), 3).to(gpu), bf16_randn((5, n_kv, d), 4).to(gpu)
    idx = torch.tensor([7, slots, -1, 2 ** 31 - 1, 0], dtype=torch.int32, device=gpu)
    print("store guard: out-of-pool slot ids are skipped", flush=True)
    store_kv_cache(kc[:slots], vc[:slots], idx, k, v)
    torch.cuda.synchronize()
    want_k = torch.zeros_like(kc)
    want_k[7], want_k[0] = k[0], k[4]
    want_v = torch.zeros_like(vc)
    want_v[7], want_v[0] = v[0], v[4]
    assert torch.equal(_bits(kc), _bits(want_k)) and torch.equal(_bits(vc), _bits(want_v))

    kc.zero_()
    vc.zero_()
    q = bf16_randn((5, 8, d), 5).to(gpu)
    w = torch.ones(d, dtype=torch.bfloat16, device=gpu)
    pos = torch.arange(5, dtype=torch.int32, device=gpu)
    q_all = qk_norm_rope_store(q, k, v, w, w, pos, idx, kc[:slots], vc[:slots], eps=1e-6, rope_base=1e4)
    good = torch.tensor([7, 1, 2, 3, 0], dtype=torch.int32, device=gpu)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    q_ref = qk_norm_rope_store(q, k, v, w, w, pos, good, kc2[:slots], vc2[:slots], eps=1e-6, rope_base=1e4)
    torch.cuda.synchronize()
    assert torch.equal(_bits(q_all), _bits(q_ref))  # q is produced for every token
    for s in (7, 0):
        assert torch.equal(_bits(kc[s]), _bits(kc2[s])) and torch.equal(_bits(vc[s]), _bits(vc2[s]))
    keep = torch.ones(slots + 8, dtype=torch.bool)
    keep[[7, 0]] = False
    assert not kc[keep.to(gpu)].any() and not vc[keep.to(gpu)].any()
