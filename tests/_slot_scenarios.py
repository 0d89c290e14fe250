"""Runs the slot-pool scenario table of tests/golden/mamba_slot_scenarios.json against a harness.

The table is data: a list of steps per scenario with the values the reference's own test file
expects (mini_sglang_mlx/tests/test_mamba_slots.py).  A harness offers
``make(num_slots, num_layers, verify_width)`` returning the pool under test plus
``fill(kind, layer, slot, value)``, ``lo / hi(kind, layer, slot)`` and ``window_shape(layer)``;
kinds are "temporal" and "conv".  Values written as "$name" refer to what an earlier step
stored under ``as``."""
import json
import os

import pytest

with open(os.path.join(os.path.dirname(__file__), "golden", "mamba_slot_scenarios.json")) as _f:
    TABLE = json.load(_f)
CONV_SHAPE = tuple(TABLE["conv_shape"])
TEMPORAL_SHAPE = tuple(TABLE["temporal_shape"])
SCENARIO_NAMES = sorted(TABLE["scenarios"])
_ERRORS = {"AssertionError": AssertionError, "RuntimeError": RuntimeError}


def run_scenario(name, harness):
    names, pool = {}, None

    def val(x):
        if isinstance(x, str) and x.startswith("$"):
            return names[x[1:]]
        if isinstance(x, list):
            return [val(e) for e in x]
        return x

    for step in TABLE["scenarios"][name]:
        op = step["op"]
        if op == "make":
            pool = harness.make(step["slots"], step.get("layers", 2), step.get("verify_width", 0))
            continue
        actions = {
            "alloc": lambda: pool.alloc(),
            "alloc_many": lambda: pool.alloc_many(step["n"]),
            "available": lambda: pool.available_size,
            "free": lambda: pool.free(val(step["slot"])),
            "free_many": lambda: pool.free_many(val(step["slots"])),
            "fill": lambda: pool.fill(step["kind"], step["layer"], val(step["slot"]), step["value"]),
            "copy": lambda: pool.copy(val(step["src"]), val(step["dst"])),
            "check_ownership": lambda: pool.check_ownership(val(step["slots"])),
            "conv_window": lambda: pool.conv_window(step["layer"]),
            "window_shape": lambda: list(pool.window_shape(step["layer"])),
            "range": lambda: (pool.lo(step["kind"], step["layer"], val(step["slot"])),
                              pool.hi(step["kind"], step["layer"], val(step["slot"]))),
        }
        if "raises" in step:
            kind, text = step["raises"]
            with pytest.raises(_ERRORS[kind], match=text) as err:
                actions[op]()
            if "message_lists" in step:
                assert f"[{val(step['message_lists'])}]" in str(err.value), (name, step)
            continue
        got = actions[op]()
        if "as" in step:
            names[step["as"]] = got
        if "expect" in step:
            assert got == val(step["expect"]), (name, step, got)
        if "expect_sorted" in step:
            want = step["expect_sorted"]
            assert (got is None) if want is None else (sorted(got) == want), (name, step, got)
        if op == "range":
            if "lo" in step:
                assert got[0] == step["lo"], (name, step, got)
            if "hi" in step:
                assert got[1] == step["hi"], (name, step, got)
