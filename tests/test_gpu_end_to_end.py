"""One layer of a serving loop, end to end on the GPU: the radix cache hands out the cached
prefix and its slots, the scheduler-side page table takes them, the metadata kernel turns the
table into CSR arrays, the fused norm + rope + store kernel writes the new tokens, the attention
operators read the pool.  A request that reuses a cached prefix must get what the same request
gets when everything is computed from scratch, and the decode steps that follow must agree
with the oracle on the gathered rows."""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import assert_close_bf16, indptr
from oracle import qk_norm_rope_oracle as qo
from test_oracle_metadata import _Req

pytestmark = pytest.mark.gpu

N_Q, N_KV, D = 16, 4, 128
VOCAB, SLOTS, MAX_SEQ = 500, 4096, 600
EPS, BASE = 1e-6, 1e6


class _Cfg:
    head_dim = D


class _Batch:
    pass


class _Layer:
    """Token-id -> raw q/k/v projections (a fixed random table, so that equal tokens give equal
    rows whichever request they sit in), the pools, the page table, the radix cache."""

    def __init__(self, gpu, seed):
        from mini_sglang_amd.attention.backend import AttnBackend
        from mini_sglang_amd.kvcache import MHAKVCache, RadixCacheManager

        g = torch.Generator().manual_seed(seed)
        r = lambda *s: torch.randn(s, generator=g).to(torch.bfloat16)
        self.emb_q, self.emb_k, self.emb_v = r(VOCAB, N_Q, D), r(VOCAB, N_KV, D), r(VOCAB, N_KV, D)
        self.qw = (1 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16)
        self.kw = (1 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16)
        self.gpu = gpu
        self.kv = MHAKVCache(num_kv_heads=N_KV, num_layers=1, head_dim=D, num_pages=SLOTS,
                             dtype=torch.bfloat16, device=gpu)
        self.page_table = torch.zeros((8, MAX_SEQ), dtype=torch.int32, device=gpu)
        self.backend = AttnBackend(_Cfg(), self.kv, self.page_table)
        self.radix = RadixCacheManager()
        self.free = torch.randperm(SLOTS, generator=g).to(torch.int32)  # scattered free slots

    def allocate(self, n):
        out, self.free = self.free[:n], self.free[n:]
        return out

    def extend(self, rows_tokens_cached):
        """One prefill step for [(table row, all tokens, cached_len)]; returns (out, reqs)."""
        reqs, new_tok, out_loc = [], [], []
        for row, tokens, cached in rows_tokens_cached:
            reqs.append(_Req(row, cached, len(tokens)))
            new_tok += tokens[cached:]
            out_loc.append(self.page_table[row, cached:len(tokens)])
        ids = torch.tensor(new_tok)
        b = _Batch()
        b.attn_metadata = self.backend.build_prefill_metadata(reqs)
        b.out_loc = torch.cat(out_loc)
        dev = lambda t: t.to(self.gpu)
        out = self.backend.forward_fused_norm_rope(
            dev(self.emb_q[ids]), dev(self.emb_k[ids]), dev(self.emb_v[ids]), dev(self.qw),
            dev(self.kw), 0, b, rms_norm_eps=EPS, rope_base=BASE)
        torch.cuda.synchronize()
        return out.float().cpu(), reqs

    def dense_reference(self, tokens, rows):
        """Attention outputs of query rows `rows` of one sequence, from the oracles alone."""
        ids = np.asarray(tokens)
        f = lambda e: e[ids].float().numpy()
        pos = np.arange(len(tokens), dtype=np.int32)
        qn = qo.rope(qo.rms_norm(f(self.emb_q), self.qw.float().numpy(), EPS), pos, BASE)
        kn = qo.rope(qo.rms_norm(f(self.emb_k), self.kw.float().numpy(), EPS), pos, BASE)
        bf = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16)
        n = len(tokens)
        q_rows = bf(qn[rows])
        want = oracle.paged_prefill_attention(
            q_rows, bf(kn), bf(f(self.emb_v)), indptr([len(rows)]), indptr([n]),
            torch.arange(n, dtype=torch.int32), torch.tensor([rows[0]], dtype=torch.int32),
            1.0 / math.sqrt(D), len(rows), return_f32=True)[1]
        return want


def test_prefix_reuse_extend_and_decode(gpu):
    rng = np.random.default_rng(11)
    layer = _Layer(gpu, seed=5)
    toks = lambda n: rng.integers(0, VOCAB, size=n).tolist()
    seq_a, seq_b = toks(150), toks(70)

    # ---- first batch: two fresh requests, prefilled together, then handed to the radix cache ----
    for row, seq in ((0, seq_a), (1, seq_b)):
        layer.page_table[row, :len(seq)] = layer.allocate(len(seq)).to(gpu)
    print("end to end: first batch", flush=True)
    out1, _ = layer.extend([(0, seq_a, 0), (1, seq_b, 0)])
    assert_close_bf16(out1[:150], layer.dense_reference(seq_a, list(range(150))), "request A")
    assert_close_bf16(out1[150:], layer.dense_reference(seq_b, list(range(70))), "request B")
    for row, seq in ((0, seq_a), (1, seq_b)):
        ids = torch.tensor(seq, dtype=torch.int32)
        assert layer.radix.insert_prefix(ids, layer.page_table[row, :len(seq)].cpu()) == 0

    # ---- second batch: C shares 97 tokens with A, D shares all of B and goes on --------------------
    seq_c = seq_a[:97] + toks(45)
    seq_d = seq_b + toks(30)
    plan = []
    for row, seq in ((2, seq_c), (3, seq_d)):
        # the last token is never matched: its logits are needed (scheduler/cache.py:30-33)
        handle, cached = layer.radix.match_prefix(torch.tensor(seq[:-1], dtype=torch.int32))
        layer.radix.lock_handle(handle)
        n = handle.cached_len
        layer.page_table[row, :n] = cached.to(gpu)
        layer.page_table[row, n:len(seq)] = layer.allocate(len(seq) - n).to(gpu)
        plan.append((row, seq, n, handle))
    assert [p[2] for p in plan] == [97, 70]
    assert layer.radix.size_info.protected_size == 97 + 70
    print("end to end: second batch (cached prefixes 97 and 70)", flush=True)
    out2, _ = layer.extend([(row, seq, n) for row, seq, n, _ in plan])
    assert_close_bf16(out2[:45], layer.dense_reference(seq_c, list(range(97, 142))), "request C on A's prefix")
    assert_close_bf16(out2[45:], layer.dense_reference(seq_d, list(range(70, 100))), "request D on B's prefix")

    # ---- decode: one more token for C and D, metadata built on the device -----------------------
    print("end to end: decode step", flush=True)
    nxt = toks(2)
    seqs = [seq_c + nxt[:1], seq_d + nxt[1:]]
    reqs = []
    for (row, _, _, _), seq in zip(plan, seqs):
        layer.page_table[row, len(seq) - 1] = layer.allocate(1).to(gpu)
        reqs.append(_Req(row, len(seq) - 1, len(seq)))
    b = _Batch()
    b.attn_metadata = layer.backend.build_decode_metadata(reqs)
    b.out_loc = torch.stack([layer.page_table[r.table_idx, r.device_len - 1] for r in reqs])
    ids = torch.tensor(nxt)
    dev = lambda t: t.to(gpu)
    out3 = layer.backend.forward_fused_norm_rope(
        dev(layer.emb_q[ids]), dev(layer.emb_k[ids]), dev(layer.emb_v[ids]), dev(layer.qw),
        dev(layer.kw), 0, b, rms_norm_eps=EPS, rope_base=BASE)
    torch.cuda.synchronize()
    for i, seq in enumerate(seqs):
        assert_close_bf16(out3[i:i + 1].float().cpu(), layer.dense_reference(seq, [len(seq) - 1]),
                          f"decode of request {i}")

    # ---- the finished requests go back to the cache; their shared prefixes are not duplicated ----
    for (row, _, n, handle), seq in zip(plan, seqs):
        ids = torch.tensor(seq, dtype=torch.int32)
        already = layer.radix.insert_prefix(ids, layer.page_table[row, :len(seq)].cpu())
        assert already == n
        layer.radix.lock_handle(handle, unlock=True)
    info = layer.radix.size_info
    assert info.protected_size == 0
    assert info.evictable_size == 150 + 70 + (len(seqs[0]) - 97) + (len(seqs[1]) - 70)
