"""bench.py's step accounting, on the CPU with a recording stand-in for the device context: exactly
--steps units are replayed inside the timed region after exactly --warmup untimed ones, whatever
their relation to the graph size, and the headline's launches never run past the problem array."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
bench = importlib.util.module_from_spec(spec)
spec.loader.exec_module(bench)


class FakeCtx:
    """Records what replay() does: graphs are lists of recorded units."""

    def __init__(self):
        self.capturing = None
        self.timing = False
        self.timed_units = 0
        self.untimed_units = 0
        self.live_graphs = 0

    def graph_begin(self):
        assert self.capturing is None
        self.capturing = []

    def graph_end(self):
        g, self.capturing = self.capturing, None
        self.live_graphs += 1
        return g

    def graph_launch(self, g):
        n = sum(c for _, c in g)
        if self.timing:
            self.timed_units += n
        else:
            self.untimed_units += n

    def graph_destroy(self, g):
        self.live_graphs -= 1

    def sync(self):
        pass

    def timer_start(self):
        self.timing = True

    def timer_stop(self):
        self.timing = False
        return 1.0


@pytest.mark.parametrize("units", [1, 2, 3, 32, 64])
@pytest.mark.parametrize("steps,warmup", [(20, 5), (1, 0), (256, 32), (257, 31), (4096, 512), (7, 300), (1000, 1)])
def test_replay_times_exactly_the_steps_asked_for(units, steps, warmup):
    ctx = FakeCtx()
    seen = []

    def record(first, n):
        assert ctx.capturing is not None and 1 <= n <= units
        assert first % units == 0          # records start at multiples of the granularity
        ctx.capturing.append((first, n))
        seen.append((first, n))

    ev, wall = bench.replay(ctx, record, units, steps, warmup)
    assert ctx.timed_units == steps and ctx.untimed_units == warmup
    assert ctx.live_graphs == 0 and ctx.capturing is None
    assert ev == pytest.approx(1.0 / steps)


def test_headline_launches_stay_inside_the_problem_array():
    # the headline alternates between gw.n // GROUP batches of GROUP problems
    n, group = 2 * bench.GROUP, bench.GROUP
    batches = n // group
    ctx = FakeCtx()
    launches = []

    def record(first, count):
        for i in range(count):
            start = ((first + i) % batches) * group
            assert 0 <= start and start + group <= n
            launches.append(start)
        ctx.capturing.append((first, count))

    bench.replay(ctx, record, batches, 20, 5)
    assert ctx.timed_units == 20 and set(launches) == {0, group}


def test_profile_facts_reads_the_machine_readable_block():
    facts = bench.profile_facts(bench.HEADLINE_PROFILE)
    assert facts["gemvs_per_launch"] == bench.GROUP
    assert facts["kernel"].startswith("gemv_t2_i8_grouped_kernel")
    algorithmic = bench.GROUP * bench.gemv_bytes(1, 4096, 11008)
    assert 0.98 < facts["traffic_bytes_per_launch"] / algorithmic < 1.05
    assert bench.profile_facts("no_such_profile.md") == {}
