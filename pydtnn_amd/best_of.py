"""Run-time choice between alternative implementations, per problem size.

Same idea and constructor as the reference's ``BestOf`` (pydtnn/utils/best_of.py:158-239): a list of
``(name, callable)`` alternatives (or ``(name, [callable per stage])`` pipelines) that take the same
arguments, and a function that maps the arguments to a hashable problem size.  Calls cycle through the
alternatives, each call is timed, alternatives slower than ``pruning_speedup`` times the best are dropped
after ``prune_after_round`` rounds, and after ``rounds`` rounds (or when one alternative is left) the one
with the smallest median time serves every later call of that problem size
(pydtnn/utils/best_of.py:308-451).  Differences, both because the work here is asynchronous GPU work:
the device is synchronised before and after a timed call (``sync``), and executions are not nested
(the reference blocks an outer BestOf while an inner one is still undecided; the alternatives here are
leaf kernels).
"""
import statistics
from collections import defaultdict
from timeit import default_timer as timer


def _default_sync():
    import torch
    if torch.cuda.is_available():
        torch.cuda.synchronize()


class BestOf:
    _use_first_alternative = False
    _instances = []

    def __init__(self, name, alternatives, get_problem_size, rounds=10, pruning_speedup=10.0, prune_after_round=4,
                 sync=None):
        assert rounds >= 1, "Rounds must be greater or equal to one."
        assert pruning_speedup > 1, "Pruning speedup must be greater than one."
        assert len(alternatives) >= 1
        first = alternatives[0][1]
        self.stages = len(first) if isinstance(first, (list, tuple)) else 1
        for alt_name, alt in alternatives:
            if self.stages == 1:
                assert callable(alt), f"Expected a function for the '{alt_name}' alternative, got a '{type(alt)}'."
            else:
                assert isinstance(alt, (list, tuple)) and len(alt) == self.stages, \
                    f"Expected {self.stages} methods for the '{alt_name}' pipeline."
        self.name = name
        self.alternatives = alternatives
        self.get_problem_size = get_problem_size
        self.total_rounds = rounds
        self.pruning_speedup = pruning_speedup
        self.prune_after_round = prune_after_round
        self.total_alternatives = len(alternatives)
        self.sync = sync if sync is not None else _default_sync
        self.best_idx = {}
        self.best_name = defaultdict(lambda: "None")
        self._current_alternative = defaultdict(int)
        self._current_round = defaultdict(int)
        self._alive = {}                                   # problem size -> indices still in the race
        self._times = defaultdict(lambda: [[] for _ in range(self.total_alternatives)])
        self._stage_times = defaultdict(lambda: [None] * self.stages)
        BestOf._instances.append(self)

    # ------------------------------------------------------------------ class-wide switches / reports
    @classmethod
    def use_always_the_first_alternative(cls, enabled=True):
        """pydtnn/utils/best_of.py:269-278: with BestOf disabled every instance just calls its first alternative."""
        cls._use_first_alternative = enabled

    @staticmethod
    def print_report():
        for inst in BestOf._instances:
            inst.print_as_table()

    # ------------------------------------------------------------------ calls
    def _method(self, idx, stage):
        alt = self.alternatives[idx][1]
        return alt if self.stages == 1 else alt[stage]

    def __call__(self, *args, **kwargs):
        args = list(args)
        stage = int(args.pop(0)) if self.stages > 1 else 0
        assert stage < self.stages, \
            f"The stage number ({stage}) must be less than the specified number of stages ({self.stages})."
        if BestOf._use_first_alternative:
            return self._method(0, stage)(*args, **kwargs)
        size = self.get_problem_size(*args, **kwargs)
        if size in self.best_idx:
            return self._method(self.best_idx[size], stage)(*args, **kwargs)
        current = self._current_alternative[size]
        self.sync()
        tic = timer()
        output = self._method(current, stage)(*args, **kwargs)
        self.sync()
        elapsed = timer() - tic
        if self.stages == 1:
            self._record(size, current, elapsed)
        else:
            # a pipeline is timed as the sum of its stages, recorded when the last stage has run after the first
            stage_times = self._stage_times[size]
            if stage == 0 or stage_times[0] is not None:
                stage_times[stage] = elapsed
            if stage == self.stages - 1 and all(t is not None for t in stage_times):
                self._record(size, current, sum(stage_times))
                self._stage_times.pop(size)
        return output

    def _record(self, size, current, elapsed):
        self._times[size][current].append(elapsed)
        alive = self._alive.setdefault(size, list(range(self.total_alternatives)))
        pos = alive.index(current)
        round_done = pos == len(alive) - 1
        next_alternative = alive[(pos + 1) % len(alive)]
        if round_done:
            self._current_round[size] += 1
            rounds = self._current_round[size]
            medians = self._medians_of(size)
            best = min(medians[i] for i in alive)
            if rounds >= min(self.prune_after_round, self.total_rounds):
                alive[:] = [i for i in alive if medians[i] <= best * self.pruning_speedup]
                next_alternative = alive[0]
            if rounds >= self.total_rounds or len(alive) == 1:
                idx = min(alive, key=lambda i: (medians[i], i))  # the first of the minima
                self.best_idx[size] = idx
                self.best_name[size] = self.alternatives[idx][0]
        self._current_alternative[size] = next_alternative

    # ------------------------------------------------------------------ queries
    def best_method_has_been_found(self, *args, **kwargs):
        return self.get_problem_size(*args, **kwargs) in self.best_idx

    def _medians_of(self, size):
        return [statistics.median(t) if t else float("nan") for t in self._times[size]]

    def medians(self):
        return {size: self._medians_of(size) for size in self._times}

    def speedups(self):
        out = {}
        for size in self._times:
            if size in self.best_idx:
                medians = [m for m in self._medians_of(size) if m == m]
                out[size] = max(medians) / self._medians_of(size)[self.best_idx[size]]
        return out

    def print_as_table(self, time_format="8.6f"):
        names = [a[0] for a in self.alternatives]
        print(f"{self.name}")
        print("  size | " + " | ".join(names) + " | speedup")
        speedups = self.speedups()
        for size, medians in self.medians().items():
            cells = []
            for i, m in enumerate(medians):
                text = format(m, time_format)
                cells.append("*" + text if self.best_idx.get(size) == i else text)
            tail = f"{speedups[size]:.1f}" if size in speedups else ""
            print(f"  {size} | " + " | ".join(cells) + " | " + tail)
