"""The shape lists of the reference's own correctness sweeps, on the GPU against the oracle.

The reference checks its kernels on one sequence of nine lengths, on single sequences with a
prefix and on ragged batches, all at head_dim 256 and four head configurations
(`mini-sglang-mlx-kernel/test_and_bench/paged_prefill_attention.py:18-25, 267-310`,
`paged_decode_attention.py:17-24, 288-309`).  Only the lists are taken from there; the inputs
are this suite's seeded workloads (random page mapping instead of the identity one)."""
import pytest

from _gpu_util import run_gpu, run_oracle
from _util import assert_close_bf16
from mini_sglang_amd.workloads import build_workload

pytestmark = pytest.mark.gpu

HEADS = [(2, 16), (4, 16), (4, 24), (2, 32)]  # (kv heads, q heads)
LENGTHS = [1, 237, 512, 809, 1024, 2048, 3333, 4096, 8192]
PREFIXED = [(237, 100), (512, 256), (1024, 512), (2048, 1024)]  # (q_len, prefix)
RAGGED_EXTENDS = [([1, 237], [0, 0]), ([512, 1024], [0, 0]), ([237, 809, 1024], [0, 100, 512]),
                  ([1, 512, 2048, 4096], [0, 0, 0, 0]), ([128, 256, 512, 1024], [64, 128, 256, 512])]
RAGGED_DECODES = [[1, 237], [512, 1024, 2048], [237, 809, 3333, 4096], [1] * 8, [4096] * 4]


def _check(wl, gpu, what):
    print(what, flush=True)
    got, _ = run_gpu(wl, gpu)
    want, _ = run_oracle(wl, precision="f32")
    return assert_close_bf16(got, want, what)


def _extend(q_lens, prefixes, n_kv, n_q, seed):
    return build_workload("r", "prefill", seed=seed, n_q=n_q, n_kv=n_kv, head_dim=256,
                          kv_lens=[p + q for p, q in zip(prefixes, q_lens)], extend_lens=q_lens,
                          pool_factor=1.2)


@pytest.mark.parametrize("n_kv,n_q", HEADS)
def test_single_sequence_extends(gpu, n_kv, n_q):
    # the longest length on the first head configuration only (the oracle's time)
    for length in LENGTHS if (n_kv, n_q) == HEADS[0] else LENGTHS[:-1]:
        _check(_extend([length], [0], n_kv, n_q, 900 + length), gpu,
               f"extend {n_kv}/{n_q} heads, one sequence of {length}")


@pytest.mark.parametrize("n_kv,n_q", HEADS)
def test_single_sequence_extends_on_a_prefix(gpu, n_kv, n_q):
    for q_len, prefix in PREFIXED:
        _check(_extend([q_len], [prefix], n_kv, n_q, 910 + q_len), gpu,
               f"extend {n_kv}/{n_q} heads, {q_len} on a prefix of {prefix}")


@pytest.mark.parametrize("n_kv,n_q", HEADS)
def test_ragged_extends(gpu, n_kv, n_q):
    for i, (q_lens, prefixes) in enumerate(RAGGED_EXTENDS):
        _check(_extend(q_lens, prefixes, n_kv, n_q, 920 + i), gpu,
               f"extend {n_kv}/{n_q} heads, q_lens {q_lens} prefixes {prefixes}")


@pytest.mark.parametrize("n_kv,n_q", HEADS)
def test_decodes(gpu, n_kv, n_q):
    for i, kv_lens in enumerate([[n] for n in LENGTHS] + RAGGED_DECODES):
        wl = build_workload("r", "decode", seed=930 + i, n_q=n_q, n_kv=n_kv, head_dim=256,
                            kv_lens=kv_lens, pool_factor=1.2)
        _check(wl, gpu, f"decode {n_kv}/{n_q} heads, kv_lens {kv_lens}")
