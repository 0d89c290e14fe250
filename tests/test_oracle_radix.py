"""The pure-Python radix oracle against the scenarios and expected values of the reference's
own tests (mini_sglang_mlx/tests/test_radix_prefix_cache.py), restated on a minimal page
allocator and slot pool (the reference drives the tree through its scheduler-side
CacheManager, scheduler/cache.py:19-76, and MambaStatePool, mamba_pool.py:107-162).
``tests/test_radix_cache.py`` runs the same scenarios on the native tree."""
import pytest

from _radix_util import (PREFIX, OraclePlain, OracleHybrid, SCENARIOS, run_scenario)


@pytest.mark.parametrize("name", sorted(SCENARIOS))
def test_reference_scenarios_on_the_oracle(name):
    run_scenario(name, OracleHybrid if SCENARIOS[name][1] else OraclePlain)


def test_fast_compare_key_known_answers():
    from oracle.radix_oracle import fast_compare_key as f

    assert f([], []) == 0 and f([1], []) == 0 and f([], [1]) == 0
    assert f([1, 2, 3], [1, 2, 3]) == 3
    assert f([1, 2, 3], [1, 2, 4]) == 2
    assert f([1, 2, 3], [1, 2]) == 2 and f([1, 2], [1, 2, 3, 4]) == 2
    assert f([5], [6]) == 0
    assert f(PREFIX, PREFIX[:3] + [9]) == 3
