"""The host half of the path checked on the machine that runs the GPU tests: the plan builder against the golden
plans and digests written by the upstream builder, against the upstream build itself where that is present, and
the device layout's lossless round trip to the upstream v2 tensors.  These are the CPU suite's checks
(test_plan_builder.py, test_plan_random.py, test_layout_host.py) run again under the `gpu` mark, because the
plan that the GPU tests and the benchmark execute is built by this machine's host cores, with this machine's
thread count."""
import pytest

pytestmark = pytest.mark.gpu

import test_layout_host as LH          # noqa: E402
import test_plan_builder as PB         # noqa: E402
import test_plan_random as PR          # noqa: E402
from helpers import golden_digests     # noqa: E402


@pytest.mark.parametrize("name", sorted(PB.CASES))
def test_golden_plans(name):
    PB.test_builder_matches_upstream_golden_plans(name)


@pytest.mark.parametrize("key", sorted(golden_digests()))
def test_golden_digests(key):
    PB.test_builder_matches_upstream_digests(key)


@pytest.mark.parametrize("name", ["toy_ps3", "rmat200_ps4", "cliques_ps3", "directed_ps3"])
def test_stepwise_api(name):
    PB.test_stepwise_api_mirrors_upstream_call_sequence(name)


def test_builder_against_the_upstream_build(oracle, capfd):
    PR.test_builder_equals_the_upstream_build_on_random_graphs(oracle, capfd)


@pytest.mark.parametrize("wl,sd,ps", [("c1", 3, 3), ("c1", 2, 2), ("c1", 3, 5), ("c3", 6, 2), ("c2", 6, 4)])
def test_layout_round_trip(wl, sd, ps):
    LH.test_layout_round_trips_to_the_upstream_v2_plan_bit_exactly(wl, sd, ps)


def test_toy_layout():
    LH.test_toy_layout_literal()
