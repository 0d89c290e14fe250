"""GDNBackend end to end on the GPU: prefill, decode, and a speculative verify window handled by
replay (copy main -> scratch, verify on the scratch slots, commit the accepted prefix to the main
slots), with the state pool holding the recurrent state.  Every state is compared with the numpy
oracle run on the same tokens (tolerance of the reference's gdn test, max-abs 5e-4)."""
import numpy as np
import pytest
import torch

from oracle import gdn_state_oracle as go

pytestmark = pytest.mark.gpu
HK, HV, D, LAYERS, WIDTH = 2, 4, 128, 2, 4
SCALE = 0.05


class _Req:
    def __init__(self, slot, extend_len):
        self.mamba_slot, self.extend_len = slot, extend_len


class _Batch:
    def __init__(self, reqs, is_decode=False):
        self.reqs, self.is_decode = reqs, is_decode
        self.mamba_slot_ids = self.mamba_prefill_indptr = None
        self.mamba_scratch_slots = self.mamba_verify_indptr = self.gdn_verify_captured = None


def _tokens(rng, n):
    f = lambda *s: go._bf16_round((SCALE * rng.standard_normal(s)).astype(np.float32))
    sig = lambda *s: go._bf16_round((1 / (1 + np.exp(-rng.standard_normal(s)))).astype(np.float32))
    return dict(q=f(n, HK, D), k=f(n, HK, D), v=f(n, HV, D), g=sig(n, HV), beta=sig(n, HV))


def _dev(gpu, d):
    return [torch.from_numpy(d[x]).to(torch.bfloat16).to(gpu) for x in ("q", "k", "v", "g", "beta")]


def _oracle(d, state, slots, indptr, single=False):
    return go.gdn_state_inplace(d["q"], d["k"], d["v"], d["g"], d["beta"], state, np.asarray(slots),
                                None if single else np.asarray(indptr, np.int32), single_token_mode=single)


def _close(got, want, what):
    diff = float(np.abs(got - want).max())
    assert diff <= 5e-4, (what, diff)


def test_prefill_decode_and_replay_style_verify(gpu):
    from mini_sglang_amd.attention import GDNBackend
    from mini_sglang_amd.kvcache import MambaStateConfig, MambaStatePool

    rng = np.random.default_rng(5)
    pool = MambaStatePool(MambaStateConfig(num_slots=8, num_layers=LAYERS, conv_shapes=[[(3, 16)]] * LAYERS,
                                           temporal_shapes=[(HV, D, D)] * LAYERS, verify_width=WIDTH),
                          device=gpu)
    backend = GDNBackend(pool)
    lengths = [5, 1, 9]
    main = [pool.alloc() for _ in lengths]
    ref = [np.zeros((9, HV, D, D), np.float32) for _ in range(LAYERS)]  # oracle copy of each layer's slab

    def check_states(what):
        torch.cuda.synchronize()
        for l in range(LAYERS):
            _close(pool.temporal_state(l).cpu().numpy(), ref[l], f"{what}, layer {l}")

    # ---- prefill: ragged extend lengths --------------------------------------------------------
    print("gdn backend: prefill", flush=True)
    batch = _Batch([_Req(s, n) for s, n in zip(main, lengths)])
    backend.prepare_batch(batch)
    assert batch.mamba_prefill_indptr.tolist() == [0, 5, 6, 15]
    for l in range(LAYERS):
        d = _tokens(rng, sum(lengths))
        y = backend.forward(*_dev(gpu, d), l, batch)
        want_y, ref[l] = _oracle(d, ref[l], main, [0, 5, 6, 15])
        _close(y.float().cpu().numpy(), want_y, f"prefill y, layer {l}")
    check_states("prefill")

    # ---- decode: one token per request ---------------------------------------------------------
    print("gdn backend: decode", flush=True)
    batch = _Batch([_Req(s, 1) for s in main], is_decode=True)
    backend.prepare_batch(batch)
    for l in range(LAYERS):
        d = _tokens(rng, len(main))
        y = backend.forward(*_dev(gpu, d), l, batch)
        want_y, ref[l] = _oracle(d, ref[l], main, None, single=True)
        _close(y.float().cpu().numpy(), want_y, f"decode y, layer {l}")
    check_states("decode")

    # ---- verify: window of WIDTH tokens per request on scratch slots ------------------------------
    print("gdn backend: verify + commit", flush=True)
    scratch = pool.alloc_many(len(main))
    pool.copy_batched(main, scratch)
    for l in range(LAYERS):
        ref[l][scratch] = ref[l][main]
    check_states("scratch seeded from main")
    batch = _Batch([_Req(s, WIDTH) for s in main])
    backend.prepare_batch(batch)
    batch.mamba_scratch_slots = torch.tensor(scratch, dtype=torch.int32, device=gpu)
    indptr = [i * WIDTH for i in range(len(main) + 1)]
    batch.mamba_verify_indptr = torch.tensor(indptr, dtype=torch.int32, device=gpu)
    window_tokens, before = [], [r.copy() for r in ref]
    for l in range(LAYERS):
        d = _tokens(rng, WIDTH * len(main))
        window_tokens.append(d)
        y = backend.forward_verify(*_dev(gpu, d), l, batch)
        want_y, ref[l] = _oracle(d, ref[l], scratch, indptr)
        _close(y.float().cpu().numpy(), want_y, f"verify y, layer {l}")
        # the conv windows a model layer would have written during the verify forward
        pool.conv_window(l, 0)[batch.mamba_scratch_slots.long()] = torch.arange(
            len(main) * WIDTH, dtype=torch.float32, device=gpu).view(len(main), WIDTH, 1, 1).expand(
            len(main), WIDTH, 3, 16).to(torch.bfloat16) + 100 * l
    check_states("verify ran on the scratch slots only")
    for l in range(LAYERS):
        np.testing.assert_array_equal(ref[l][main], before[l][main])

    accepted = [2, 0, 3]  # drafts accepted per request: replay 3, 1 and 4 tokens
    backend.commit_verify(batch, accepted)
    assert batch.gdn_verify_captured is None
    for l in range(LAYERS):
        d = window_tokens[l]
        keep = np.concatenate([np.arange(i * WIDTH, i * WIDTH + j + 1) for i, j in enumerate(accepted)])
        sub = {x: d[x][keep] for x in d}
        lens = [j + 1 for j in accepted]
        _, ref[l] = _oracle(sub, ref[l], main, np.concatenate([[0], np.cumsum(lens)]))
    check_states("accepted prefixes replayed into the main slots")
    for l in range(LAYERS):
        conv = pool.conv_state(l, 0).float().cpu()
        for i, (slot, j) in enumerate(zip(main, accepted)):
            assert float(conv[slot].min()) == float(conv[slot].max()) == i * WIDTH + j + 100 * l

    with pytest.raises(ValueError, match="accepted counts"):
        batch.gdn_verify_captured = {0: _dev(gpu, window_tokens[0])}
        backend.commit_verify(batch, [WIDTH, 0, 0])
    pool.free_many(scratch)
    for s in main:
        pool.free(s)
    pool.check_ownership([])
