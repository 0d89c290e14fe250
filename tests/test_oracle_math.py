"""Pins the oracle's attention values against mathematics it does not share code with:
an independent numpy float64 softmax-attention, closed forms, and invariants of the path
chosen so that a dropped term, an off-by-one in a mask bound, a wrong kv-head mapping or a
wrong merge weight fails at least one of them."""
import math

import numpy as np
import pytest
import torch

import oracle
from _util import bf16_randn, dense_attention_f64, indptr

D = 128
SCALE = 1.0 / math.sqrt(D)


def make_case(seed, extend_lens, prefixes, n_q=4, n_kv=2, slots_extra=5):
    kv_lens = [p + e for p, e in zip(prefixes, extend_lens)]
    total_kv = sum(kv_lens)
    g = torch.Generator().manual_seed(seed)
    num_slots = total_kv + slots_extra
    perm = torch.randperm(num_slots, generator=g)[:total_kv].to(torch.int32)
    return dict(
        q=bf16_randn((sum(extend_lens), n_q, D), seed + 1),
        k_cache=bf16_randn((num_slots, n_kv, D), seed + 2),
        v_cache=bf16_randn((num_slots, n_kv, D), seed + 3),
        qo_indptr=indptr(extend_lens), kv_indptr=indptr(kv_lens), kv_indices=perm,
        prefix_lens=torch.tensor(prefixes, dtype=torch.int32),
        max_len_extend=max(extend_lens), kv_lens=kv_lens)


def run_prefill(c, **kw):
    return oracle.paged_prefill_attention(
        c["q"], c["k_cache"], c["v_cache"], c["qo_indptr"], c["kv_indptr"], c["kv_indices"],
        c["prefix_lens"], SCALE, c["max_len_extend"], return_f32=True, **kw)[1]


@pytest.mark.parametrize("is_cross,window", [(False, 0), (True, 0), (False, 3), (True, 3),
                                             (False, 1), (False, 64)])
def test_prefill_equals_textbook_float64(is_cross, window):
    c = make_case(11, extend_lens=[5, 1, 9, 3], prefixes=[7, 0, 20, 33], n_q=6, n_kv=3)
    got = run_prefill(c, is_cross_attention=is_cross, sliding_window_size=window)
    want = dense_attention_f64(c["q"], c["k_cache"], c["v_cache"], c["qo_indptr"],
                               c["kv_indptr"], c["kv_indices"], c["prefix_lens"], SCALE,
                               is_cross, window)
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=0, atol=2e-6)


def test_decode_equals_textbook_and_prefill_qlen1():
    kv_lens = [1, 31, 32, 33, 129, 300]
    c = make_case(21, extend_lens=[1] * 6, prefixes=[l - 1 for l in kv_lens], n_q=8, n_kv=2)
    splits = torch.tensor([min(32, max(1, (l + 127) // 128)) for l in kv_lens], dtype=torch.int32)
    dec = oracle.paged_decode_attention(c["q"], c["k_cache"], c["v_cache"], c["kv_indptr"],
                                        c["kv_indices"], splits, SCALE, 32, return_f32=True)[1]
    want = dense_attention_f64(c["q"], c["k_cache"], c["v_cache"], c["qo_indptr"],
                               c["kv_indptr"], c["kv_indices"], c["prefix_lens"], SCALE)
    np.testing.assert_allclose(dec.numpy(), want.numpy(), rtol=0, atol=2e-6)
    pre = run_prefill(c)
    np.testing.assert_allclose(dec.numpy(), pre.numpy(), rtol=0, atol=2e-6)


@pytest.mark.parametrize("splits", [1, 2, 3, 7, 32])
def test_decode_is_split_invariant_and_merge_is_the_closed_form(splits):
    kv_lens = [257, 64, 1000]
    c = make_case(31, extend_lens=[1] * 3, prefixes=[l - 1 for l in kv_lens])
    base = oracle.paged_decode_attention(
        c["q"], c["k_cache"], c["v_cache"], c["kv_indptr"], c["kv_indices"],
        torch.ones(3, dtype=torch.int32), SCALE, 32, return_f32=True)[1]
    sp = torch.full((3,), splits, dtype=torch.int32)
    out, att_out, att_lse = oracle.paged_decode_attention(
        c["q"], c["k_cache"], c["v_cache"], c["kv_indptr"], c["kv_indices"], sp, SCALE, 32,
        return_f32=True, return_partials=True)[1:]
    np.testing.assert_allclose(out.numpy(), base.numpy(), rtol=0, atol=3e-6)
    # closed form of the merge: o = sum_s exp(lse_s - LSE) * O_s over the non-empty splits
    for b, L in enumerate(kv_lens):
        per = oracle.decode_kv_len_per_split(L, splits)
        n_used = sum(1 for s in range(splits) if per * s < L)
        lse = att_lse[b, :, :n_used].double()
        w = torch.softmax(lse, dim=-1)
        merged = (w[..., None] * att_out[b, :, :n_used].double()).sum(1)
        np.testing.assert_allclose(merged.numpy(), base[b].double().numpy(), rtol=0, atol=3e-6)


def test_split_geometry_formula_exhaustive():
    # paged_decode_attention.metal:356-362: splits tile [0, L) exactly, lengths are
    # multiples of 32 except the last, and empty splits only trail
    for L in list(range(1, 200)) + [1023, 1024, 1025, 4097]:
        for splits in range(1, 33):
            per = oracle.decode_kv_len_per_split(L, splits)
            assert per % 32 == 0 and per * splits >= L
            assert per == ((-(-L // splits)) + 31) // 32 * 32
            covered, seen_empty = 0, False
            for s in range(splits):
                lo, hi = per * s, min(per * s + per, L)
                if lo >= hi:
                    seen_empty = True
                    continue
                assert not seen_empty and lo == covered
                covered = hi
            assert covered == L


def test_window_at_least_kv_len_equals_no_window_and_cross_qlen1_equals_causal():
    c = make_case(41, extend_lens=[6, 2], prefixes=[10, 0])
    a = run_prefill(c)
    b = run_prefill(c, sliding_window_size=max(c["kv_lens"]))
    assert torch.equal(a, b)
    c1 = make_case(42, extend_lens=[1, 1], prefixes=[9, 30])
    assert torch.equal(run_prefill(c1), run_prefill(c1, is_cross_attention=True))


def test_one_extend_equals_two_chunked_extends():
    # a 12-token extend == a 5-token extend followed by a 7-token extend on prefix + 5
    c = make_case(51, extend_lens=[12], prefixes=[9])
    full = run_prefill(c)
    idx = c["kv_indices"]
    first = dict(c, q=c["q"][:5], qo_indptr=indptr([5]), kv_indptr=indptr([14]),
                 kv_indices=idx[:14], prefix_lens=torch.tensor([9], dtype=torch.int32),
                 max_len_extend=5)
    second = dict(c, q=c["q"][5:], qo_indptr=indptr([7]), kv_indptr=indptr([21]),
                  kv_indices=idx, prefix_lens=torch.tensor([14], dtype=torch.int32),
                  max_len_extend=7)
    got = torch.cat([run_prefill(first), run_prefill(second)])
    np.testing.assert_allclose(got.numpy(), full.numpy(), rtol=0, atol=1e-6)


def test_slot_permutation_and_batch_order_leave_outputs_unchanged():
    c = make_case(61, extend_lens=[3, 4], prefixes=[5, 2])
    base = run_prefill(c)
    n = c["k_cache"].shape[0]
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(5))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(n)
    moved = dict(c, k_cache=c["k_cache"][perm], v_cache=c["v_cache"][perm],
                 kv_indices=inv[c["kv_indices"].long()].to(torch.int32))
    assert torch.equal(run_prefill(moved), base)
    # swap the two requests
    kv = c["kv_indptr"].tolist()
    swapped = dict(
        c, q=torch.cat([c["q"][3:], c["q"][:3]]), qo_indptr=indptr([4, 3]),
        kv_indptr=indptr([6, 8]),
        kv_indices=torch.cat([c["kv_indices"][kv[1]:], c["kv_indices"][:kv[1]]]),
        prefix_lens=torch.tensor([2, 5], dtype=torch.int32))
    out = run_prefill(swapped)
    assert torch.equal(torch.cat([out[4:], out[:4]]), base)


def test_gqa_head_mapping_constant_v_dominant_key_and_masked_rows():
    c = make_case(71, extend_lens=[4], prefixes=[6], n_q=6, n_kv=2)
    # q heads of one kv group given identical rows produce identical outputs, and the
    # group is h // (n_q / n_kv): heads 0..2 -> kv 0, 3..5 -> kv 1
    q = c["q"].clone()
    q[:, 1] = q[:, 0]
    q[:, 2] = q[:, 0]
    q[:, 4] = q[:, 0]
    out = run_prefill(dict(c, q=q))
    assert torch.equal(out[:, 0], out[:, 1]) and torch.equal(out[:, 0], out[:, 2])
    assert not torch.equal(out[:, 0], out[:, 4])
    # V constant per kv head => output equals that constant
    vconst = c["v_cache"].clone()
    vconst[:, 0] = 0.5
    vconst[:, 1] = -2.0
    out = run_prefill(dict(c, v_cache=vconst))
    np.testing.assert_allclose(out[:, :3].numpy(), 0.5, atol=1e-6)
    np.testing.assert_allclose(out[:, 3:].numpy(), -2.0, atol=1e-6)
    # one key with a huge score => output is that key's V row
    kdom = c["k_cache"].clone()
    slot = int(c["kv_indices"][2])
    kdom[slot, 0] = (c["q"][0, 0].float() * 50).to(torch.bfloat16)
    out = run_prefill(dict(c, k_cache=kdom))
    np.testing.assert_allclose(out[0, 0].numpy(), c["v_cache"][slot, 0].float().numpy(), atol=1e-5)
    # rows without any visible key are exact zeros: kv stream shorter than the prefix
    short = dict(c, kv_indptr=indptr([3]), kv_indices=c["kv_indices"][:3],
                 prefix_lens=torch.tensor([6], dtype=torch.int32))
    out = run_prefill(short, sliding_window_size=2)
    assert torch.count_nonzero(out) == 0


def test_bf16_rounding_is_round_to_nearest_even_like_torch():
    x = torch.randn(4096, generator=torch.Generator().manual_seed(3)) * 37.0
    x = torch.cat([x, torch.tensor([0.0, -0.0, 1.00390625, 1.01171875, 3.3895e38, 1e-40])])
    bits = oracle.f32_to_bf16_bits(x.numpy())
    want = x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(bits, want)
    back = oracle.bf16_bits_to_f32(bits)
    assert np.array_equal(back, x.to(torch.bfloat16).float().numpy())


def test_f32_build_agrees_with_f64_build():
    c = make_case(81, extend_lens=[7, 3], prefixes=[40, 11], n_q=8, n_kv=2)
    a = run_prefill(c)
    b = oracle.paged_prefill_attention(
        c["q"], c["k_cache"], c["v_cache"], c["qo_indptr"], c["kv_indptr"], c["kv_indices"],
        c["prefix_lens"], SCALE, c["max_len_extend"], precision="f32", return_f32=True)[1]
    np.testing.assert_allclose(a.numpy(), b.numpy(), rtol=0, atol=5e-6)
