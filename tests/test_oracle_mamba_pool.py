"""The state-pool oracle against the reference's own slot-lifecycle scenarios."""
import numpy as np
import pytest

from _slot_scenarios import CONV_SHAPE, SCENARIO_NAMES, TEMPORAL_SHAPE, run_scenario
from oracle.mamba_pool_oracle import MambaPoolOracle

_BF16 = {0.0: 0x0000, 3.0: 0x4040, 5.0: 0x40A0, 7.0: 0x40E0}  # bit patterns of the values used


class _OraclePool(MambaPoolOracle):
    def _buf(self, kind, layer):
        return self.temporal[layer] if kind == "temporal" else self.conv[layer][0]

    def fill(self, kind, layer, slot, value):
        self._buf(kind, layer)[slot] = value if kind == "temporal" else _BF16[value]

    def _values(self, kind, layer, slot):
        raw = self._buf(kind, layer)[slot]
        if kind == "temporal":
            return raw
        back = {v: k for k, v in _BF16.items()}
        return np.vectorize(back.__getitem__)(raw)

    def lo(self, kind, layer, slot):
        return float(self._values(kind, layer, slot).min())

    def hi(self, kind, layer, slot):
        return float(self._values(kind, layer, slot).max())

    def window_shape(self, layer):
        return self.conv_window(layer).shape


class OracleHarness:
    @staticmethod
    def make(num_slots, num_layers=2, verify_width=0):
        return _OraclePool(num_slots, num_layers, [[CONV_SHAPE]] * num_layers,
                           [TEMPORAL_SHAPE] * num_layers, verify_width)


@pytest.mark.parametrize("scenario", SCENARIO_NAMES)
def test_reference_scenarios(scenario):
    run_scenario(scenario, OracleHarness)


def test_copy_batched_reads_every_source_before_it_writes():
    pool = OracleHarness.make(4)
    for slot in range(1, 5):
        pool.temporal[0][slot] = float(slot)
    pool.copy_batched([1, 2], [2, 3])  # slot 2 is a source and a destination
    assert [float(pool.temporal[0][s].max()) for s in range(1, 5)] == [1.0, 1.0, 2.0, 4.0]
