"""The scenario simulator on the CPU, against the stand-in device of the scheduler's tests: what it draws, that a
healthy engine passes, and that each of the engine's test-only bugs is caught (the reference sweeps its own faults
the same way: sim/simulate.cpp:283-300, README.md:86-93)."""

import pytest

from bitwise_amd.config.engine import EngineConfig, Fault
from bitwise_amd.sim import KINDS, Simulator
from fake_executor import FakeExecutor


def stand_in(cfg: EngineConfig) -> FakeExecutor:
    return FakeExecutor(cfg.block_size, max_model_len=cfg.max_model_len or (1 << 20), run_ahead=cfg.run_ahead)


def simulator(fault: int = 0) -> Simulator:
    return Simulator(None, "bfloat16", executor_factory=stand_in, fault=fault, max_len=400)


def test_a_scenario_is_a_function_of_its_seed_and_draws_the_engines_own_knobs():
    sim = simulator()
    a, b = sim.draw(12345), sim.draw(12345)
    assert a.describe() == b.describe() and [x.prompt for x in a.arrivals] == [x.prompt for x in b.arrivals]
    seen = {"page": set(), "graphs": set(), "ahead": set(), "kind": set(), "exact_len": 0, "waves": set()}
    for seed in range(300):
        sc = sim.draw(seed)
        e = sc.engine
        e.validate()
        seen["page"].add(e.block_size), seen["graphs"].add(e.use_graphs), seen["ahead"].add(e.run_ahead), seen["kind"].add(sc.kind)
        longest = max(len(x.prompt) + x.params.max_new_tokens for x in sc.arrivals)
        assert longest <= e.max_model_len <= 400 and e.num_blocks * e.block_size >= longest + 1
        seen["exact_len"] += int(e.max_model_len == longest)
        if sc.kind == "waves":
            sizes = {}
            for x in sc.arrivals:
                sizes[x.at_step] = sizes.get(x.at_step, 0) + 1
            seen["waves"].add(tuple(sizes[k] for k in sorted(sizes)))
    assert seen["page"] == {8, 16, 32, 64} and seen["graphs"] == {True, False} and seen["ahead"] == {True, False}
    assert seen["kind"] == set(KINDS) and seen["exact_len"] > 30
    assert (1, 2, 4, 8) in seen["waves"] and (1, 2) in seen["waves"]          # the waves double: every graph bucket up to 8


def test_a_healthy_engine_passes_and_the_scenarios_reach_what_they_are_built_for():
    tally = simulator().run(200, seed=3)
    assert tally.violations() == 0, "\n".join(tally.notes[:5])
    assert tally.requests_compared > 500
    assert tally.preemptions > 0 and tally.prefix_hit_tokens > 0 and tally.ended_by_eos > 0 and tally.cancelled > 0
    assert tally.knobs_seen["block_size"] == {8, 16, 32, 64} and tally.knobs_seen["kind"] == set(KINDS)
    assert tally.line("x").startswith("x: 200 scenarios") and "first failing" not in tally.line("x")


@pytest.mark.parametrize("fault", sorted(Fault.NAMES))
def test_every_injected_fault_is_caught(fault):
    tally = simulator(fault).run(120, seed=3)
    assert tally.violations() > 0 and tally.first_failing >= 0, Fault.NAMES[fault]
    assert "first failing scenario" in tally.line(Fault.NAMES[fault])


def test_the_oracle_never_carries_the_fault():
    sim = simulator(Fault.RNG_KEYED_BY_STEP)
    from bitwise_amd.config.engine import SamplingParams
    sp = SamplingParams(temperature=0.9, seed=4, max_new_tokens=12, ignore_eos=True)
    assert sim.solo([5, 6, 7], sp) == simulator().solo([5, 6, 7], sp)
