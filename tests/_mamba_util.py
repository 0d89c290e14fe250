"""The scenarios of the reference's mini_sglang_mlx/tests/test_mamba_slots.py, restated with their
expected values and run against a harness: the numpy oracle on the CPU, the GPU pool on the GPU.
A harness offers ``make(num_slots, num_layers=2, verify_width=0)`` returning an object with the
pool's methods plus ``fill(kind, layer, slot, value)``, ``lo(kind, layer, slot)``,
``hi(kind, layer, slot)`` and ``window_shape(layer)``; kinds are "temporal" and "conv"."""
import pytest

CONV_SHAPE = (3, 4)         # (state_len, d_inner), _factories.py:20
TEMPORAL_SHAPE = (2, 3, 4)  # (num_heads, head_dim, state_size), _factories.py:21


def alloc_is_lifo_and_never_hands_out_slot_zero(h):
    pool = h.make(3)
    assert pool.available_size == 3
    assert [pool.alloc() for _ in range(3)] == [3, 2, 1]
    assert pool.available_size == 0
    assert pool.alloc() is None


def free_makes_the_slot_available_again_most_recently_first(h):
    pool = h.make(2)
    first, second = pool.alloc(), pool.alloc()
    pool.free(first)
    assert pool.alloc() == first
    pool.free(second)
    assert pool.alloc() == second


def alloc_zeroes_the_state_it_hands_out(h):
    pool = h.make(1)
    slot = pool.alloc()
    pool.fill("temporal", 0, slot, 5.0)
    pool.fill("conv", 0, slot, 5.0)
    assert pool.lo("temporal", 0, slot) == 5.0
    pool.free(slot)
    assert pool.alloc() == slot
    assert pool.hi("temporal", 0, slot) == 0.0 and pool.lo("temporal", 0, slot) == 0.0
    assert pool.hi("conv", 0, slot) == 0.0 and pool.lo("conv", 0, slot) == 0.0


def alloc_many_refuses_without_consuming_anything(h):
    pool = h.make(2)
    assert pool.alloc_many(3) is None
    assert pool.available_size == 2
    assert sorted(pool.alloc_many(2)) == [1, 2]
    assert pool.available_size == 0
    assert pool.alloc_many(0) == []


def double_free_is_rejected(h):
    pool = h.make(2)
    slot = pool.alloc()
    pool.free(slot)
    with pytest.raises(AssertionError, match="already free"):
        pool.free(slot)
    slots = pool.alloc_many(2)
    pool.free_many(slots)
    assert pool.available_size == 2
    with pytest.raises(AssertionError, match="already free"):
        pool.free_many(slots)


def free_rejects_slots_outside_the_pool(h):
    for slot in (0, -1, 3):
        pool = h.make(2)
        with pytest.raises(AssertionError, match="Invalid slot"):
            pool.free(slot)


def check_ownership_accepts_a_free_list_and_tree_slots(h):
    pool = h.make(3)
    in_tree = pool.alloc()
    pool.check_ownership([in_tree])
    pool.free(in_tree)
    pool.check_ownership([])


def check_ownership_reports_a_slot_nobody_owns(h):
    pool = h.make(3)
    leaked = pool.alloc()
    with pytest.raises(RuntimeError) as err:
        pool.check_ownership([])
    assert "leaked" in str(err.value)
    assert f"[{leaked}]" in str(err.value)
    pool.free(leaked)
    pool.check_ownership([])


def check_ownership_rejects_one_slot_owned_twice(h):
    pool = h.make(2)
    slot = pool.alloc()
    pool.free(slot)
    with pytest.raises(AssertionError, match="owned twice"):
        pool.check_ownership([slot])


def copy_duplicates_state_without_aliasing_the_source(h):
    pool = h.make(2)
    src, dst = pool.alloc(), pool.alloc()
    pool.fill("temporal", 1, src, 7.0)
    pool.fill("conv", 1, src, 3.0)
    pool.copy(src, dst)
    assert pool.lo("temporal", 1, dst) == 7.0 and pool.hi("temporal", 1, dst) == 7.0
    assert pool.lo("conv", 1, dst) == 3.0 and pool.hi("conv", 1, dst) == 3.0
    # layer 0 was zero in both and stays so
    assert pool.hi("temporal", 0, dst) == 0.0
    pool.fill("temporal", 1, dst, 0.0)
    assert pool.lo("temporal", 1, src) == 7.0


def conv_window_buffers_follow_verify_width(h):
    plain = h.make(1, verify_width=0)
    with pytest.raises(AssertionError, match="conv windows not allocated"):
        plain.conv_window(0)
    verifier = h.make(1, verify_width=4)
    assert verifier.window_shape(0) == (2, 4, *CONV_SHAPE)  # (slots + padding slot, steps, ...)


SCENARIOS = [
    alloc_is_lifo_and_never_hands_out_slot_zero,
    free_makes_the_slot_available_again_most_recently_first,
    alloc_zeroes_the_state_it_hands_out,
    alloc_many_refuses_without_consuming_anything,
    double_free_is_rejected,
    free_rejects_slots_outside_the_pool,
    check_ownership_accepts_a_free_list_and_tree_slots,
    check_ownership_reports_a_slot_nobody_owns,
    check_ownership_rejects_one_slot_owned_twice,
    copy_duplicates_state_without_aliasing_the_source,
    conv_window_buffers_follow_verify_width,
]
