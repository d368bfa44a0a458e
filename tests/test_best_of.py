"""BestOf (pydtnn_amd/best_of.py) on the CPU: fake alternatives whose "run time" is a counter, so that the
selection logic of pydtnn/utils/best_of.py:308-451 can be checked without a GPU or real timing."""
import pytest


class Clock:
    """Replaces timeit's timer inside best_of: each alternative advances it by a fixed amount."""

    def __init__(self):
        self.now = 0.0

    def __call__(self):
        return self.now


@pytest.fixture
def best_of(monkeypatch):
    from pydtnn_amd import best_of as mod
    clock = Clock()
    monkeypatch.setattr(mod, "timer", clock)
    mod.BestOf.use_always_the_first_alternative(False)
    yield mod.BestOf, clock
    mod.BestOf.use_always_the_first_alternative(False)


def make(clock, cost, log, name):
    def f(x):
        clock.now += cost
        log.append(name)
        return (name, x)
    return f


def test_picks_the_fastest_after_the_rounds(best_of):
    BestOf, clock = best_of
    log = []
    b = BestOf("t", [("slow", make(clock, 3.0, log, "slow")), ("fast", make(clock, 1.0, log, "fast")),
                     ("mid", make(clock, 2.0, log, "mid"))], get_problem_size=lambda x: x, rounds=3,
               sync=lambda: None)
    for _ in range(9):
        assert not b.best_method_has_been_found(7)
        b(7)
    assert log == ["slow", "fast", "mid"] * 3
    assert b.best_method_has_been_found(7) and b.best_name[7] == "fast"
    assert b(7) == ("fast", 7) and b(7) == ("fast", 7)
    assert b.medians()[7] == [3.0, 1.0, 2.0] and b.speedups()[7] == 3.0
    # another problem size starts its own race
    assert b(8) == ("slow", 8) and not b.best_method_has_been_found(8)


def test_prunes_hopeless_alternatives(best_of):
    BestOf, clock = best_of
    log = []
    b = BestOf("t", [("awful", make(clock, 100.0, log, "awful")), ("a", make(clock, 1.0, log, "a")),
                     ("b", make(clock, 1.5, log, "b"))], get_problem_size=lambda x: 0, rounds=6,
               pruning_speedup=10.0, prune_after_round=2, sync=lambda: None)
    for _ in range(6 + 2 * 4):
        b(0)
    assert log.count("awful") == 2 and b.best_name[0] == "a"


def test_single_survivor_ends_the_race_early(best_of):
    BestOf, clock = best_of
    log = []
    b = BestOf("t", [("x", make(clock, 50.0, log, "x")), ("y", make(clock, 1.0, log, "y"))],
               get_problem_size=lambda x: 0, rounds=10, pruning_speedup=2.0, prune_after_round=1, sync=lambda: None)
    b(0), b(0)
    assert b.best_method_has_been_found(0) and b.best_name[0] == "y"


def test_pipeline_is_timed_as_the_sum_of_its_stages(best_of):
    BestOf, clock = best_of
    log = []
    # alternative p: cheap forward, expensive backward; q: the other way round but cheaper in all
    p = [make(clock, 1.0, log, "p0"), make(clock, 5.0, log, "p1")]
    q = [make(clock, 2.0, log, "q0"), make(clock, 2.0, log, "q1")]
    b = BestOf("t", [("p", p), ("q", q)], get_problem_size=lambda x: 0, rounds=2, sync=lambda: None)
    for _ in range(4):
        b(0, "x")
        b(1, "y")
    assert log == ["p0", "p1", "q0", "q1"] * 2          # a backward always follows its own forward
    assert b.best_name[0] == "q" and b.medians()[0] == [6.0, 4.0]
    assert b(0, 1) == ("q0", 1) and b(1, 2) == ("q1", 2)
    with pytest.raises(AssertionError):
        b(2, 0)


def test_disabled_means_first_alternative(best_of):
    BestOf, clock = best_of
    log = []
    b = BestOf("t", [("first", make(clock, 9.0, log, "first")), ("second", make(clock, 1.0, log, "second"))],
               get_problem_size=lambda x: 0, sync=lambda: None)
    BestOf.use_always_the_first_alternative()
    for _ in range(30):
        b(0)
    assert set(log) == {"first"} and not b.best_method_has_been_found(0)
