"""Plans chosen by measurement.  The parts that can do a product in several ways (the package's weight-streaming
kernel with one or four tiles per wavefront and K in 1 to 16 parts, the BLAS library with K whole or in pieces side by
side, ...) decide by rules that were measured at the layer sizes of a few models (kernels/tuning.py).  For other sizes,
or simply to be sure, the runner can measure instead, before it records a step of some number of rows:

  1. the step runs once with `collecting()` on: every product that has more than one plan reports its key (kind of
     product, class of its row count, sizes, flags) and operands through `choose`, and runs by the rules;
  2. `tune` times each candidate plan of each new key on the device, as replays of a recorded graph that walks the
     weights of all layers that reported the key (so that no weight is cache-resident, as in a real step), with the
     consumer that pays for the plan's output format (the norm that adds partial sums) included, and keeps the fastest;
  3. from then on `choose` answers with the kept plan for that key.

A plan decides speed only: every candidate computes the same product with 32-bit accumulation, so results differ in
rounding at most.  The kept plans live in a `Table` that belongs to the runner that measured them (a second runner
may be handed the same table); `choose` answers from the table that is in use (`using(table)`, which the runner puts
around every forward), so a runner built without autotune runs by the rules whatever other runners of the process have
measured.  A key is measured when a step with it is about to be recorded, the second time the step's sizes are seen:
the first step of those sizes has run by the rules, so in bfloat16 a runner with autotune gives up the promise that a
step's bits do not depend on whether its sizes have been seen before (the plans differ in rounding).
"""
import contextlib
import sys
import time

import torch

class Table(dict):
    """key -> kept plan; `report` lists (key, chosen plan, {plan: microseconds}) of every key measured into it."""

    def __init__(self):
        super().__init__()
        self.report = []


KINDS = {}            # kind of product -> ProductKind
_collected = None     # while collecting: key -> list of operand tuples
_current = None       # the table in use (a runner's, around its forward), or None: by the rules
MAX_ROTATION = 32     # weights that a timing graph walks through
FLUSH_BYTES = 1 << 29 # written before every timed replay: more than the caches hold, so that every weight comes from memory
MARGIN = 0.10         # a plan must beat the rules' plan by this fraction to replace it: the timing stands for the step only so far


class ProductKind:
    """How the tuner handles one kind of product: `candidates(key)` lists plans, the first being the plan the rules
    give; `make(key, operands_list, device)` returns a function run(plan, i) that does the product with the i-th
    operands (and whatever consumes its output format)."""

    def __init__(self, candidates, make):
        self.candidates, self.make = candidates, make


def register_kind(name, candidates, make):
    KINDS[name] = ProductKind(candidates, make)


@contextlib.contextmanager
def collecting():
    """Products report their keys and operands while this is on, and run by the rules."""
    global _collected
    prev, _collected = _collected, {}
    try:
        yield _collected
    finally:
        _collected = prev


@contextlib.contextmanager
def using(table):
    """The products inside run by the plans of `table` (None: by the rules)."""
    global _current
    prev, _current = _current, table
    try:
        yield table
    finally:
        _current = prev


def choose(key, operands):
    """The kept plan for `key` in the table in use, or None (run by the rules).  `operands` is remembered while
    collecting."""
    if _collected is not None:
        seen = _collected.setdefault(key, [])
        if len(seen) < 4 * MAX_ROTATION:
            seen.append(operands)
        return None
    return _current.get(key) if _current is not None else None


def rows_class(rows):
    """Row counts share a plan in classes: up to 16 rows each count by itself, beyond that the multiples of 16 stand for
    the counts below them (a plan is timed at the class's own count; 64, the most rows that the weight-streaming kernel
    takes, ends a class)."""
    return rows if rows <= 16 else -(-rows // 16) * 16


def active():
    return bool(_current) or _collected is not None


def _graph_time(run, n, flush, replays=5):
    """Microseconds per call of run(i), i = 0..n-1, from replays of a graph that holds the n calls; before each
    replay `flush` is overwritten, which empties the caches of what the replay before left there."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(n):
            run(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(n):
            run(i)
    graph.replay()
    torch.cuda.synchronize()
    best = None
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        flush.add_(1)
        e0.record()
        graph.replay()
        e1.record()
        e1.synchronize()
        t = e0.elapsed_time(e1) * 1e3 / n
        best = t if best is None else min(best, t)
    del graph
    return best


def tune(collected, device, table, verbose=False):
    """Measures the candidate plans of every collected key that `table` has no plan for yet, and keeps the fastest
    there.  Returns the number of keys measured."""
    done = 0
    flush = None
    for key, operands_list in collected.items():
        if key in table or key[0] not in KINDS:
            continue
        kind = KINDS[key[0]]
        plans = kind.candidates(key)
        if len(plans) < 2:
            table[key] = plans[0] if plans else None
            continue
        # the operands of different layers, one of each (by the address of the first tensor)
        unique, seen = [], set()
        for ops_ in operands_list:
            at = ops_[0].data_ptr()
            if at not in seen:
                seen.add(at)
                unique.append(ops_)
        unique = unique[:MAX_ROTATION]
        t0 = time.perf_counter()
        if flush is None:
            flush = torch.zeros((FLUSH_BYTES // 4,), dtype=torch.int32, device=device)
        run = kind.make(key, unique, device)
        times = {}
        for plan in plans:
            try:
                times[plan] = _graph_time(lambda i: run(plan, i), len(unique), flush)
            except Exception as e:              # a candidate that the kernels refuse is no candidate
                torch.cuda.synchronize()
                if verbose:
                    sys.stderr.write("[ginfer_amd] autotune %s: plan %s refused (%s)\n" % (key, plan, e))
        if not times:
            continue
        by_rules = plans[0]
        best = min(times, key=times.get)
        if by_rules in times and times[best] > times[by_rules] * (1.0 - MARGIN):
            best = by_rules
        table[key] = best
        table.report.append((key, best, times))
        done += 1
        if verbose:
            sys.stderr.write("[ginfer_amd] autotune %s: %s %.1f us (rules: %s %.1f us; %d plans in %.2f s)\n"
                             % (key, best, times[best], by_rules, times.get(by_rules, float("nan")), len(times),
                                time.perf_counter() - t0))
    return done
