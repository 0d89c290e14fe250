"""The GPU state pool: the reference's slot-lifecycle scenarios on the real class, and its
copies and zero fills bit for bit against the numpy oracle."""
import numpy as np
import pytest
import torch

from _slot_scenarios import CONV_SHAPE, SCENARIO_NAMES, TEMPORAL_SHAPE, run_scenario
from mini_sglang_amd.kvcache import (MambaStateConfig, MambaStatePool,
                                     create_hybrid_radix_cache_manager)
from oracle.mamba_pool_oracle import MambaPoolOracle

pytestmark = pytest.mark.gpu


class _GpuPool(MambaStatePool):
    def _buf(self, kind, layer):
        return self.temporal_state(layer) if kind == "temporal" else self.conv_state(layer, 0)

    def fill(self, kind, layer, slot, value):
        self._buf(kind, layer)[slot] = value

    def lo(self, kind, layer, slot):
        return float(self._buf(kind, layer)[slot].float().min())

    def hi(self, kind, layer, slot):
        return float(self._buf(kind, layer)[slot].float().max())

    def window_shape(self, layer):
        return tuple(self.conv_window(layer).shape)


class GpuHarness:
    device = None

    @classmethod
    def make(cls, num_slots, num_layers=2, verify_width=0):
        return _GpuPool(MambaStateConfig(num_slots=num_slots, num_layers=num_layers,
                                         conv_shapes=[[CONV_SHAPE] for _ in range(num_layers)],
                                         temporal_shapes=[TEMPORAL_SHAPE] * num_layers,
                                         dtype=torch.float32, verify_width=verify_width),
                        device=cls.device)


@pytest.mark.parametrize("scenario", SCENARIO_NAMES)
def test_reference_scenarios(gpu, scenario):
    GpuHarness.device = gpu
    print(scenario, flush=True)
    run_scenario(scenario, GpuHarness)


def _random_pools(gpu, num_slots, layers, conv_shapes, temporal_shapes, seed):
    """A GPU pool and an oracle pool holding the same random bits."""
    cfg = MambaStateConfig(num_slots=num_slots, num_layers=layers, conv_shapes=conv_shapes,
                           temporal_shapes=temporal_shapes)
    pool = MambaStatePool(cfg, device=gpu)
    ref = MambaPoolOracle(num_slots, layers, conv_shapes, temporal_shapes)
    g = torch.Generator().manual_seed(seed)
    for l in range(layers):
        t = torch.randn(ref.temporal[l].shape, generator=g)
        ref.temporal[l][...] = t.numpy()
        pool.temporal_state(l).copy_(t)
        for c in range(len(conv_shapes[l])):
            bits = torch.randint(0, 1 << 15, ref.conv[l][c].shape, generator=g, dtype=torch.int32)
            ref.conv[l][c][...] = bits.numpy().astype(np.uint16)
            pool.conv_state(l, c).view(torch.int16).copy_(bits.to(torch.int16))
    return pool, ref


def _assert_same(pool, ref):
    for l in range(ref.num_layers):
        got = pool.temporal_state(l).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), ref.temporal[l].view(np.uint32)), f"temporal layer {l}"
        for c in range(len(ref.conv[l])):
            got = pool.conv_state(l, c).view(torch.int16).cpu().numpy().view(np.uint16)
            assert np.array_equal(got, ref.conv[l][c]), f"conv layer {l} group {c}"


@pytest.mark.parametrize("seed", range(6))
def test_copies_and_zero_fills_match_the_oracle_bit_for_bit(gpu, seed):
    rng = np.random.default_rng(seed)
    layers = int(rng.integers(1, 5))
    # layers of two different shapes (two slabs per kind), odd row lengths (narrow accesses),
    # rows longer than one 16 KiB piece
    shapes_t = [(2, 3, 4), (4, 64, 40)] if seed % 2 else [(3, 5, 7), (8, 128, 16)]
    shapes_c = [[(3, 4)], [(3, 5), (4, 33)]]
    temporal = [shapes_t[l % 2] for l in range(layers)]
    conv = [shapes_c[l % 2] for l in range(layers)]
    slots = int(rng.integers(4, 12))
    pool, ref = _random_pools(gpu, slots, layers, conv, temporal, seed)
    print(f"state pool seed={seed} layers={layers} slots={slots}", flush=True)
    _assert_same(pool, ref)
    for _ in range(8):
        ids = rng.permutation(np.arange(0, slots + 1))
        n = int(rng.integers(1, (slots + 1) // 2 + 1))
        src, dst = ids[:n].tolist(), ids[n:2 * n].tolist()
        if rng.random() < 0.5:
            pool.copy_batched(src, dst)
        else:  # ids already on the device, as the engine passes them
            pool.copy_batched(torch.tensor(src, dtype=torch.int32, device=gpu),
                              torch.tensor(dst, dtype=torch.int32, device=gpu))
        ref.copy_batched(src, dst)
        slot = int(rng.integers(1, slots + 1))
        pool._zero_slot(slot)
        for buf in ref._state_buffers():
            buf[slot] = 0
        pool.copy(slot, slot)  # a no-op
    torch.cuda.synchronize()
    _assert_same(pool, ref)


def test_copy_batched_refuses_overlapping_host_ids_and_skips_ids_outside_the_pool(gpu):
    pool, ref = _random_pools(gpu, 4, 2, [[(3, 4)]] * 2, [(2, 3, 4)] * 2, 11)
    with pytest.raises(ValueError, match="distinct"):
        pool.copy_batched([1, 2], [2, 3])
    with pytest.raises(ValueError, match="distinct"):
        pool.copy_batched([1, 2], [3, 3])
    # device ids cannot be checked on the host: ids outside the pool are skipped by the kernel
    pool.copy_batched(torch.tensor([1, 99, -3], dtype=torch.int32, device=gpu),
                      torch.tensor([2, 3, 4], dtype=torch.int32, device=gpu))
    ref.copy_batched([1], [2])
    torch.cuda.synchronize()
    _assert_same(pool, ref)


def test_pool_is_the_state_of_the_gdn_kernel_and_the_slot_source_of_the_hybrid_cache(gpu):
    """The pool's temporal slab view goes straight into gdn_state_inplace; its slots are what the
    hybrid radix manager frees on eviction."""
    from mini_sglang_amd_kernel import gdn_state_inplace

    hk, hv, d = 2, 4, 128
    pool = MambaStatePool(MambaStateConfig(num_slots=3, num_layers=2, conv_shapes=[[(3, 8)]] * 2,
                                           temporal_shapes=[(hv, d, d)] * 2), device=gpu)
    slot = pool.alloc()
    g = torch.Generator().manual_seed(3)
    q = torch.randn(1, hk, d, generator=g).to(gpu, torch.bfloat16)
    k = torch.randn(1, hk, d, generator=g).to(gpu, torch.bfloat16)
    v = torch.randn(1, hv, d, generator=g).to(gpu, torch.bfloat16)
    gate = (-torch.rand(1, hv, generator=g)).to(gpu, torch.bfloat16)
    beta = torch.rand(1, hv, generator=g).to(gpu, torch.bfloat16)
    state = pool.temporal_state(1)
    assert state.is_contiguous() and state.shape == (4, hv, d, d)
    print("gdn on a pool slot", flush=True)
    gdn_state_inplace(q, k, v, gate, beta, state, torch.tensor([slot], dtype=torch.int32, device=gpu),
                      torch.tensor([0, 1], dtype=torch.int32, device=gpu), single_token_mode=True)
    torch.cuda.synchronize()
    assert float(state[slot].abs().max()) > 0 and float(pool.temporal_state(0)[slot].abs().max()) == 0
    snapshot = pool.alloc()
    pool.copy(slot, snapshot)
    assert torch.equal(state[snapshot], state[slot])
    manager = create_hybrid_radix_cache_manager(pool)
    ids = torch.arange(16, dtype=torch.int32)
    manager.insert_prefix(ids, torch.arange(16, dtype=torch.int32), mamba_slot=snapshot)
    pool.free(slot)
    manager.check_integrity()  # free list + tree own every slot
    manager.evict(16)
    assert pool.available_size == 3
