"""Variant search for the autograd functions of the path: grid or random search over a
function's search space, each point timed by the function's own ``build_and_test``.

Same entry point as the reference (tuning/my_autograd_func_tuner.py:14-68), which delegates the
search to SparTA's ``GridSearchTuner`` / ``RandomSearchTuner``; those are restated here in a few
lines each, since what they do for this path is enumerate points and keep the fastest.  The
reference's ``build_and_test`` never returns a latency (its timing is a TODO), so its tuner could
not rank anything; here every trial yields milliseconds, failed trials are logged and skipped.
"""
from __future__ import annotations

import itertools
import logging
import math
import random
from typing import Any, Callable, Optional

from ..pytorch.cpp_extensions.layers_and_funcs.utils import MyAutogradFunc, TunableItemCfg

_logger = logging.getLogger(__name__)


class Tuner:
    """Evaluates up to ``max_trials`` points of ``search_space`` with ``eval_func(index, point)``
    (milliseconds; an exception marks the trial as failed) and keeps the fastest."""

    def __init__(self, search_space: dict[str, TunableItemCfg], eval_func: Callable[[int, dict], float],
                 max_trials: int):
        self.search_space = search_space
        self.eval_func = eval_func
        self.max_trials = max_trials
        self.best_config: Optional[dict[str, Any]] = None
        self.best_latency = math.inf
        self.trials: list[tuple[dict, Optional[float]]] = []

    def size(self) -> int:
        return math.prod(len(item._value) for item in self.search_space.values())

    def point(self, index: int) -> dict[str, Any]:
        """Point ``index`` of the grid in row-major order (the last parameter varies fastest)."""
        out = {}
        for name in reversed(list(self.search_space)):
            choices = self.search_space[name]._value
            index, i = divmod(index, len(choices))
            out[name] = choices[i]
        return {name: out[name] for name in self.search_space}

    def indices(self):
        raise NotImplementedError

    def tune(self) -> Optional[dict[str, Any]]:
        for trial, index in enumerate(itertools.islice(self.indices(), self.max_trials)):
            params = self.point(index)
            try:
                latency = float(self.eval_func(trial, params))
            except Exception as e:  # a variant that cannot run these operands
                _logger.info("trial %d %s failed: %s", trial, params, e)
                self.trials.append((params, None))
                continue
            self.trials.append((params, latency))
            if latency < self.best_latency:
                self.best_latency, self.best_config = latency, params
        return self.best_config


class GridSearchTuner(Tuner):
    def indices(self):
        return iter(range(self.size()))


class RandomSearchTuner(Tuner):
    """Distinct points in random order (seeded: the same seed visits the same points)."""

    def __init__(self, search_space, eval_func, max_trials, seed: int = 0):
        super().__init__(search_space, eval_func, max_trials)
        self.seed = seed

    def indices(self):
        rng = random.Random(self.seed)
        size = self.size()
        if size <= 1 << 16:
            order = list(range(size))
            rng.shuffle(order)
            return iter(order)
        seen: set[int] = set()

        def draw():
            while len(seen) < size:
                i = rng.randrange(size)
                if i not in seen:
                    seen.add(i)
                    yield i
        return draw()


def tune_my_autograd_function(autograd_func: type[MyAutogradFunc], name: str, sample_inputs: list,
                              sample_grads: Optional[list] = None, algo: str = "grid", max_trials: int = 40,
                              seed: int = 0, return_tuner: bool = False):
    """Best point of ``autograd_func.get_search_space(...)`` by measured forward + backward time
    on the sample operands, or None when every trial failed."""
    if algo.startswith("grid"):
        make = GridSearchTuner
    elif algo.startswith("rand"):
        make = lambda *a: RandomSearchTuner(*a, seed=seed)  # noqa: E731
    else:
        raise ValueError(f'unsupported tuner algorithm "{algo}"')
    space = autograd_func.get_search_space(sample_inputs, sample_grads)

    def evaluate(trial: int, params: dict) -> float:
        latency = autograd_func.build_and_test(sample_inputs, sample_grads, params)
        _logger.info("[%s] #%d %s: %.4f ms", name, trial, params, latency)
        return latency

    tuner = make(space, evaluate, max_trials)
    tuner.max_trials = min(max_trials, tuner.size())
    tuner.tune()
    if tuner.best_config is None:
        _logger.warning("[%s] All trials failed.", name)
    else:
        _logger.info("[%s] Best config: %s (%.4f ms)", name, tuner.best_config, tuner.best_latency)
    return tuner if return_tuner else tuner.best_config
