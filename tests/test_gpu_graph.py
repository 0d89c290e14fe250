"""A decode step captured once in a HIP graph and replayed: the library's entry points neither
allocate nor synchronise nor read sizes back from the device, so a serving loop can record
(metadata build -> fused norm + rope + store -> decode attention) and replay it with new inputs
in the same buffers.  Every replay is checked against the same step run eagerly on a second
set of pools, with eager work and synchronisations between the replays."""
import math

import pytest
import torch

from mini_sglang_amd_kernel import (build_attention_metadata, paged_decode_attention,
                                    paged_prefill_attention, qk_norm_rope_store)

pytestmark = pytest.mark.gpu

N_Q, N_KV, D = 16, 4, 128
BATCH, MAX_SEQ, SLOTS = 6, 512, 4096
EPS, BASE = 1e-6, 1e6


class _State:
    """Everything a decode step touches, in fixed buffers."""

    def __init__(self, gpu, seed):
        g = torch.Generator().manual_seed(seed)
        bf = lambda *s: torch.randn(s, generator=g).to(gpu, torch.bfloat16)
        self.k_cache, self.v_cache = bf(SLOTS, N_KV, D), bf(SLOTS, N_KV, D)
        self.qw = (1 + 0.1 * torch.randn(D, generator=g)).to(gpu, torch.bfloat16)
        self.kw = (1 + 0.1 * torch.randn(D, generator=g)).to(gpu, torch.bfloat16)
        perm = torch.randperm(SLOTS, generator=g)[:BATCH * MAX_SEQ].to(torch.int32)
        self.page_table = perm.view(BATCH, MAX_SEQ).to(gpu)
        self.table_rows = torch.tensor([3, 0, 5, 1, 4, 2], dtype=torch.int32, device=gpu)
        self.kv_lens = torch.tensor([17, 300, 64, 1, 129, 255], dtype=torch.int32, device=gpu)
        self.q = torch.zeros(BATCH, N_Q, D, dtype=torch.bfloat16, device=gpu)
        self.k = torch.zeros(BATCH, N_KV, D, dtype=torch.bfloat16, device=gpu)
        self.v = torch.zeros(BATCH, N_KV, D, dtype=torch.bfloat16, device=gpu)
        self.out = torch.zeros(BATCH, N_Q, D, dtype=torch.bfloat16, device=gpu)

    def step(self):
        """One decode step of one layer: every request grows by the token in q / k / v."""
        self.kv_lens.add_(1)
        meta = build_attention_metadata(self.page_table, self.table_rows, self.kv_lens,
                                        total_kv=BATCH * MAX_SEQ)
        out_loc = self.page_table[self.table_rows.long(), (self.kv_lens - 1).long()]
        q_rot = qk_norm_rope_store(self.q, self.k, self.v, self.qw, self.kw, meta["positions"], out_loc,
                                   self.k_cache, self.v_cache, eps=EPS, rope_base=BASE)
        res = paged_decode_attention(q_rot, self.k_cache, self.v_cache, meta["kv_indptr"],
                                     meta["kv_indices"], meta["num_kv_splits"], 1.0 / math.sqrt(D), 32)
        self.out.copy_(res)


def test_decode_step_replays_from_a_graph(gpu):
    torch.cuda.set_device(gpu)
    captured, eager = _State(gpu, 21), _State(gpu, 21)
    g = torch.Generator().manual_seed(22)
    tokens = [[torch.randn(s, generator=g).to(torch.bfloat16) for s in
               ((BATCH, N_Q, D), (BATCH, N_KV, D), (BATCH, N_KV, D))] for _ in range(7)]

    def feed(state, i):
        for dst, src in zip((state.q, state.k, state.v), tokens[i]):
            dst.copy_(src.to(gpu))

    # warm-up on a side stream (first calls load the library and fill the allocator's pools)
    side = torch.cuda.Stream(device=gpu)
    side.wait_stream(torch.cuda.current_stream(gpu))
    with torch.cuda.stream(side):
        feed(captured, 0)
        captured.step()
    torch.cuda.current_stream(gpu).wait_stream(side)
    torch.cuda.synchronize()
    feed(eager, 0)
    eager.step()
    torch.cuda.synchronize()
    assert torch.equal(captured.out, eager.out)

    print("capturing a decode step", flush=True)
    graph = torch.cuda.CUDAGraph()
    feed(captured, 1)
    with torch.cuda.graph(graph):
        captured.step()
    # capture records, it does not run: the lengths move when the graph is replayed
    captured.kv_lens.copy_(eager.kv_lens)
    for i in range(1, 7):
        print(f"replay {i}", flush=True)
        feed(captured, i)
        graph.replay()
        torch.cuda.synchronize()
        feed(eager, i)
        eager.step()
        torch.cuda.synchronize()
        assert torch.equal(captured.kv_lens, eager.kv_lens)
        assert torch.equal(captured.out.view(torch.int16), eager.out.view(torch.int16)), f"replay {i}"
        assert torch.equal(captured.k_cache.view(torch.int16), eager.k_cache.view(torch.int16))
        # unrelated eager work between replays (its allocations must not disturb the graph's)
        junk = torch.randn(1 << 20, device=gpu).sum()
        assert torch.isfinite(junk)


def test_extend_with_key_splits_replays_from_a_graph(gpu):
    """The tile kernels with a key split (partials in a workspace, then the merge kernel) and the
    short-query split-K route, captured and replayed on changing inputs."""
    from mini_sglang_amd.workloads import build_workload

    torch.cuda.set_device(gpu)
    for extend in (40, 6):
        wl = build_workload("t", "prefill", seed=31, n_q=N_Q, n_kv=N_KV, head_dim=D,
                            kv_lens=[9000 + extend], extend_lens=[extend], pool_factor=1.1)
        w = wl.to(gpu)
        run = lambda: paged_prefill_attention(w.q, w.k_cache, w.v_cache, w.qo_indptr, w.kv_indptr,
                                              w.kv_indices, w.prefix_lens, w.sm_scale, extend)
        want = run()
        torch.cuda.synchronize()
        out = torch.zeros_like(want)
        print(f"capturing an extend of {extend} tokens", flush=True)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out.copy_(run())
        for i in range(4):
            if i:  # new queries in the same buffer
                w.q.copy_(torch.randn(w.q.shape, generator=torch.Generator().manual_seed(40 + i)).to(gpu))
                want = run()
                torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), want.view(torch.int16)), f"extend {extend} replay {i}"
