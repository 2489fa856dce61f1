"""Training a branched graph (graph.Tape) under a device-memory budget.

The reference's swapping executors decide per tensor of the dataflow graph what leaves the device
after its forward use and comes back before its backward use (python/athena/gpu_ops/
vdnnExecutor.py:202-330: offload on one copy stream, prefetch on another, DLEventRecord /
DLEventSync around every move; the policy switch of examples/imagenet_resnet.py:139-154).  This
module does that for the tape of graph.py, which runs the residual, multi-branch and attention
graphs of the reference's examples:

  record(build)       runs the graph builder without arithmetic and returns, per operator call, the
                      size of its output, what it read, and what its backward operators read again;
  plan(record, ...)   replays the executor's schedule on those sizes and, while the replayed peak
                      exceeds the budget, takes the largest value that sits idle at the moment of the
                      peak off the device (greedy, as planner.py does for layer lists): the output of
                      an operator that is cheap to run again (BatchNorm, Relu, add, scale, concat: one
                      to three passes over HBM) is dropped and computed again when the backward sweep
                      needs it, any other value is sent to pinned host memory;
  BudgetedTape        a Tape that follows the plan: values without a later reader are dropped as the
                      forward sweep passes their last use, values to be computed again likewise,
                      values sent away go to pinned host memory behind the sweep (keeping their memory
                      for `hold` more operators, while the copy runs) and are fetched `lead` operators
                      ahead of the backward sweep, and every value is dropped after the last backward
                      operator (or recomputation) that reads it;
  BudgetedRun         trains step after step under a plan; BudgetedRun.tune runs a few steps under each
                      of several (lead, hold) schedules and keeps the fastest;
  plan_split          when moving and recomputing whole values cannot meet the budget (one operator's
                      operands, results and gradients do not fit), the END of the graph - from some
                      operator on, up to the loss - runs per batch micro-tensor (graph.MicroTape: forward
                      and backward of one micro-tensor back to back, so that stretch's values and
                      gradients exist for one micro-tensor at a time); the planner takes the shortest
                      such stretch under which the rest can be planned, measuring what a stretch holds by
                      running it on a backend that only counts bytes (measure_tail).

Schedule (replayed byte for byte by `replay`, measured against the pool by the tests):
  forward  of operator t : its output is allocated; then every value whose last reader in the forward
                           sweep was t and which no backward operator reads is released; a planned
                           value whose last forward reader was t starts leaving, and is released
                           after operator t + hold has been issued (the host waits for the copy then,
                           if it is still on its way);
  backward of operator j : the values sent away that operators j - lead .. j need first (in the order
                           of the sweep) are allocated and start coming back; the host waits for
                           those operator j reads; dropped values operator j needs first are computed
                           again, producers before consumers (a Relu output from the BatchNorm output
                           from the kept convolution output), which gives the same bits; j's backward
                           operators allocate the gradients of its inputs; then j's output gradient
                           and every value whose last reader was j are released.
Ordering between the streams goes through the host (DLEventRecord / DLEventQuery / DLEventSync), as in
the reference: a value's copy out is issued once the operator that last read it has run, a copy back
once everything that was in flight when its memory was taken from the pool has run (so that no kernel
reads memory the pool has handed out again).  The executor looks at those events as the sweeps pass
and issues the copies that have become ready; the host waits only when a copy's time has come (a value
due for release, or one its reader needs) and it has not been issued or has not finished.  With `hold`
and `lead` of a few dozen operators the copies run beside the operators instead of between them; the
memory that costs is part of the replay, so the planner makes room for it by sending more away.
Which (lead, hold) is fastest depends on the graph and the budget: BudgetedRun.tune measures.

The budget covers what the tape allocates: operator outputs, gradients, parameters and their
gradients, inputs and constants.  The operator library's own scratch is outside it.
"""
import collections

import numpy as np

from . import graph
from . import ndarray
from .stream import create_event_handle, create_stream_handle


def _bytes(shape):
    n = 4
    for s in shape:
        n *= int(s)
    return n


class OpRecord(object):
    """One operator call of a recorded graph.  Indices refer to operator calls (-1: a leaf)."""
    __slots__ = ["bytes", "inputs", "saved", "has_backward", "grad_inputs", "leaf_grad_bytes", "cheap", "name",
                 "transient", "early_grads", "early_leaf_grad_bytes"]

    def __init__(self, nbytes, inputs, saved, has_backward, grad_inputs, leaf_grad_bytes, cheap=False, name=None):
        self.name = name                   # the Tape method of the call
        # a stretch of operators run per micro-tensor (split_tail): bytes it holds on top of its inputs while it
        # runs, the outside values whose gradients it leaves behind, and the parameter gradients it creates
        self.transient, self.early_grads, self.early_leaf_grad_bytes = 0, (), 0
        self.cheap = cheap                 # the operator can compute its output again from its inputs
        self.bytes = nbytes                # of the output
        self.inputs = inputs               # producers of the values the forward operator reads
        self.saved = saved                 # producers of the values the backward operators read
        self.has_backward = has_backward
        self.grad_inputs = grad_inputs     # producers of the inputs that receive a gradient (operator outputs only)
        self.leaf_grad_bytes = leaf_grad_bytes   # bytes of parameter gradients this operator's backward creates


_ShapeOnly = graph._ShapeOnly


class _Zeros(object):
    trainable = {}

    def get(self, name, shape, init, trainable=True):
        return np.broadcast_to(np.float32(0), tuple(int(s) for s in shape))


def record(build, inputs, fuse_bn_relu=False):
    """Runs `build(tape, binder, cache)` (as graphbench.py's builders: cache maps input names to Vars)
    on shapes only.  inputs: name -> shape.  -> (list of OpRecord, bytes of the leaves: inputs,
    parameters, constants).  fuse_bn_relu: the builders' BatchNorm + Relu pairs are one node each."""
    from .workloads import ShapeBinder
    t = graph.Tape(_ShapeOnly())
    t.fuse_bn_relu = fuse_bn_relu
    t._log = []
    b = ShapeBinder(t, _Zeros())
    cache = {k: t.const(None, shape) for k, shape in inputs.items()}
    loss, _ = build(t, b, cache)
    assert len(t._log) == len(t._nodes)          # every operator call is one node
    ops = []
    seen_param_grads = set()
    for node, call in zip(t._nodes, t._log):
        leaf_grad = 0
        for v in node.inputs:
            if v.node < 0 and v.needs_grad and node.back is not None and id(v) not in seen_param_grads:
                seen_param_grads.add(id(v))
                leaf_grad += _bytes(v.shape)
        ops.append(OpRecord(_bytes(node.out.shape), [v.node for v in node.inputs], [v.node for v in node.saved],
                            node.back is not None,
                            [v.node for v in node.inputs if v.node >= 0 and v.needs_grad] if node.back is not None else [],
                            leaf_grad, node.redo is not None, call[0]))
    leaves = sum(_bytes(s) for s in inputs.values()) + sum(_bytes(v.shape) for v in b.vars.values())
    leaves += sum(_bytes(shape) for _, shape in b._consts.values())
    assert loss.node == len(ops) - 1
    return ops, leaves


class TapePlan(object):
    def __init__(self, away, lead, peak_bytes, free_peak_bytes, budget_bytes, leaves_bytes, redo=(), hold=1):
        self.away = frozenset(away)          # operator calls whose output leaves the device between the sweeps
        self.redo = frozenset(redo)          # operator calls whose output is dropped and computed again
        self.lead = lead                     # operators ahead of its first reader at which a value starts coming back
        self.hold = hold                     # operators behind its last reader after which a leaving value is released
        self.peak_bytes = peak_bytes
        self.free_peak_bytes = free_peak_bytes     # replayed peak with nothing sent away
        self.budget_bytes = budget_bytes
        self.leaves_bytes = leaves_bytes
        self.split_from, self.pieces = None, 1   # plan_split: operators from split_from on run per micro-tensor

    def describe(self):
        gib = float(1 << 30)
        return {"away": len(self.away), "recomputed": len(self.redo), "lead": self.lead, "hold": self.hold,
                "peak_GiB": self.peak_bytes / gib,
                "unplanned_peak_GiB": self.free_peak_bytes / gib,
                "budget_GiB": None if self.budget_bytes is None else self.budget_bytes / gib,
                "split_from": self.split_from, "pieces": self.pieces}


def _uses(ops):
    """last forward reader and the backward readers of every operator's output"""
    n = len(ops)
    last_fwd = list(range(n))                 # at least its own producer
    bwd = [[] for _ in range(n)]
    for t, op in enumerate(ops):
        for i in op.inputs:
            if i >= 0:
                last_fwd[i] = max(last_fwd[i], t)
        if op.has_backward:
            for i in op.saved:
                if i >= 0:
                    bwd[i].append(t)
    return last_fwd, bwd


def _needs(ops, redo):
    """When, in the backward sweep, every value must be on the device: need[i] lists the operators
    during whose backward step value i is read - by their backward operators, or by the recomputation
    of a dropped value, which happens in the step of that value's first reader.  The sweep descends,
    so max(need[i]) is the first moment and min(need[i]) the last."""
    last_fwd, bwd = _uses(ops)
    need = [list(r) for r in bwd]
    for c in sorted(redo, reverse=True):      # consumers before producers
        if not need[c]:
            continue                          # nobody reads it again: it is simply dropped
        t = max(need[c])
        for u in set(ops[c].inputs):
            if u >= 0:
                need[u].append(t)
    return last_fwd, need


def replay(ops, leaves_bytes, away=(), lead=3, redo=(), hold=1):
    """Peak of the executor's schedule with `away` sent to the host and `redo` dropped and computed
    again.  -> (peak bytes, moment of the peak, values resident and idle at that moment: list of
    (bytes, operator)).  A moment is an operator index for the forward sweep and 2n - 1 - j for the
    backward step of operator j."""
    n = len(ops)
    away, redo = set(away), set(redo)
    last_fwd, need = _needs(ops, redo)
    first = [max(r) if r else -1 for r in need]
    last = [min(r) if r else -1 for r in need]
    live = leaves_bytes
    resident = {}                                       # operator -> bytes of its value on the device
    peak, peak_at, peak_set = live, -1, []
    busy = set()

    def note(moment):
        nonlocal peak, peak_at, peak_set
        if live > peak:
            peak, peak_at = live, moment
            peak_set = [(b, i) for i, b in resident.items() if i not in busy]

    by_last_fwd = collections.defaultdict(list)
    for i in range(n):
        by_last_fwd[last_fwd[i]].append(i)
    leaving = []                                        # (operator after which it is released, value)
    # ---- forward
    grads = {}                                          # operator -> bytes of the gradient of its output
    for t, op in enumerate(ops):
        live += op.bytes
        resident[t] = op.bytes
        busy = set(i for i in op.inputs if i >= 0) | {t}
        note(t)
        if op.transient:
            # a stretch run per micro-tensor: what one piece holds at its worst moment, then the
            # gradients it leaves behind (of outside values, released as the backward sweep passes their
            # producers, and of parameters)
            live += op.transient
            note(t)
            live -= op.transient
            for i in op.early_grads:
                grads[i] = ops[i].bytes
                live += ops[i].bytes
            live += op.early_leaf_grad_bytes
            note(t)
        for due, i in leaving:
            if due <= t:
                live -= resident.pop(i)
        leaving = [(due, i) for due, i in leaving if due > t]
        for i in by_last_fwd[t]:
            if not need[i] or i in redo:
                if i != n - 1:                          # the loss stays for the caller
                    live -= resident.pop(i)
            elif i in away:
                leaving.append((t + hold, i))
    for due, i in leaving:
        live -= resident.pop(i)
    # ---- backward
    fetch_at = collections.defaultdict(list)
    for i in away:
        if need[i]:
            fetch_at[min(n - 1, first[i] + lead)].append(i)
    redo_at = collections.defaultdict(list)
    for i in redo:
        if need[i]:
            redo_at[first[i]].append(i)
    by_last = collections.defaultdict(list)
    for i in range(n):
        if need[i]:
            by_last[last[i]].append(i)
    for j in range(n - 1, -1, -1):
        op = ops[j]
        moment = 2 * n - 1 - j
        for i in sorted(fetch_at[j], key=lambda i: -first[i]):
            if i not in resident:
                live += ops[i].bytes
                resident[i] = ops[i].bytes
        busy = set(i for i in op.saved if i >= 0)
        for i in sorted(redo_at[j]):                    # producers before consumers
            busy |= set(u for u in ops[i].inputs if u >= 0) | {i}
            if i not in resident:
                live += ops[i].bytes
                resident[i] = ops[i].bytes
                note(moment)
        note(moment)
        if op.has_backward and (j == n - 1 or j in grads):
            # every input that takes a gradient gets a new array; adding to an earlier one holds the
            # sum and both terms for a moment
            for i in op.grad_inputs:
                extra = ops[i].bytes
                live += extra
                if i in grads:
                    live += extra
                    note(moment)
                    live -= 2 * extra
                else:
                    grads[i] = extra
                note(moment)
            live += op.leaf_grad_bytes
            note(moment)
        if j in grads:
            live -= grads.pop(j)
        for i in by_last[j]:
            if i in resident:
                live -= resident.pop(i)
    return peak, peak_at, peak_set


def plan(ops, leaves_bytes, budget_bytes, lead=3, min_bytes=1 << 20, recompute=True, hold=1):
    """-> TapePlan.  Raises ValueError when the budget cannot be met (a single operator's operands,
    results and gradients do not fit with everything idle off the device)."""
    free_peak, _, _ = replay(ops, leaves_bytes, (), lead, (), hold)
    away, redo, banned = set(), set(), set()
    n = len(ops)
    if budget_bytes is not None:
        while True:
            peak, at, idle = replay(ops, leaves_bytes, away, lead, redo, hold)
            if peak <= budget_bytes:
                break
            last_fwd, need = _needs(ops, redo)
            # values that could be off the device at that moment: read again only later in the backward
            # sweep, after a gap
            cands = []
            for b, i in idle:
                if i in away or i in redo or not need[i] or b < min_bytes:
                    continue
                gone_from = last_fwd[i] + 1
                cheap = recompute and ops[i].cheap and (i, "redo") not in banned
                back_at = 2 * n - 1 - (max(need[i]) if cheap else min(n - 1, max(need[i]) + lead))
                if not cheap:
                    gone_from += hold                   # a copy takes that many more operators to leave
                    if (i, "away") in banned:
                        continue
                if gone_from <= at < back_at:
                    cands.append((b, i, cheap))
            if not cands:
                raise ValueError("a step does not fit %.2f GiB: %.2f GiB are needed at once with everything "
                                 "idle off the device" % (budget_bytes / float(1 << 30), peak / float(1 << 30)))
            # a value that can be computed again goes before one that has to travel, the larger first
            b, i, cheap = max(cands, key=lambda c: (c[2], c[0], c[1]))
            trial_away, trial_redo = (away, redo | {i}) if cheap else (away | {i}, redo)
            new_peak, new_at, _ = replay(ops, leaves_bytes, trial_away, lead, trial_redo, hold)
            if new_peak > peak or (new_peak == peak and new_at == at):
                # keeping this value's inputs for the recomputation (or the move itself) does not help
                # here: try the other way, then other values
                banned.add((i, "redo" if cheap else "away"))
                continue
            away, redo = set(trial_away), set(trial_redo)
    peak, _, _ = replay(ops, leaves_bytes, away, lead, redo, hold)
    return TapePlan(away, lead, peak, free_peak, budget_bytes, leaves_bytes, redo, hold)


def first_splittable(ops):
    """Smallest operator index from which on no operator couples the samples of a batch: a stretch
    run per micro-tensor may start there or later."""
    s = len(ops) - 1
    while s > 0 and ops[s - 1].name not in graph.COUPLES_SAMPLES:
        s -= 1
    return s


def split_tail(ops, split_from, transient_bytes):
    """The recorded graph with the operators from `split_from` on as ONE operator, run per micro-tensor
    with forward and backward back to back (graph.MicroTape): it reads the outside values the stretch
    reads, its output is the loss, nothing is kept for the backward sweep, and while it runs it holds
    `transient_bytes` (measure_tail) on top of them; the gradients of the outside values and of the
    stretch's parameters exist from then on."""
    tail = ops[split_from:]
    assert tail and ops[-1].name == "softmax_ce" and not any(op.name in graph.COUPLES_SAMPLES for op in tail)
    outside = sorted({i for op in tail for i in op.inputs if 0 <= i < split_from})
    sup = OpRecord(ops[-1].bytes, outside, [], False, [], 0, False, "micro_tensor_tail")
    sup.transient = int(transient_bytes)
    sup.early_grads = tuple(sorted({i for op in tail for i in op.grad_inputs if 0 <= i < split_from}))
    sup.early_leaf_grad_bytes = sum(op.leaf_grad_bytes for op in tail)
    return list(ops[:split_from]) + [sup]


class _Counter(object):
    def __init__(self):
        self.live = self.peak = 0


class _FakeArray(object):
    """Stands for a device array of `nbytes`: counted while it is referenced, as the pool counts the real one."""
    __slots__ = ["nbytes", "counter", "owner"]

    def __init__(self, nbytes, counter, owner=None):
        self.nbytes, self.counter, self.owner = nbytes, counter, owner
        counter.live += nbytes
        counter.peak = max(counter.peak, counter.live)

    def __del__(self):
        self.counter.live -= self.nbytes


class _NoLinks(object):
    def __getattr__(self, name):
        return lambda *a, **k: None


class CountingBackend(graph.GpuBackend):
    """graph.GpuBackend with every library call taken out: the same Python runs, allocating and dropping
    stand-in arrays at the same points, so the bytes a tape holds can be read off without a device."""
    L = _NoLinks()

    def __init__(self):
        self.ctx, self.stream, self.counter = None, None, _Counter()

    def empty(self, shape):
        return _FakeArray((_bytes(shape) + 255) // 256 * 256, self.counter)

    def from_numpy(self, a):
        return self.empty(np.shape(a))

    def piece(self, x, pieces, index):
        return _FakeArray(0, self.counter, x)            # a view: no memory of its own, keeps its parent

    def assign(self, dst, src):
        pass

    def sync(self):
        pass


def measure_tail(build, inputs, piece_calls, split_from, pieces, fuse_bn_relu=False):
    """Bytes the stretch of operators from `split_from` on holds at its worst moment, beyond what is
    resident when it starts, when run per micro-tensor: found by running the builder on a MicroTape over
    a backend that only counts (the executor's own Python, stand-in arrays)."""
    from .workloads import ShapeBinder
    backend = CountingBackend()
    level = {}

    class Probe(graph.MicroTape):
        def _run_pieces(self, loss_var):
            level["start"] = backend.counter.live
            backend.counter.peak = backend.counter.live
            out = graph.MicroTape._run_pieces(self, loss_var)
            level["peak"] = backend.counter.peak
            return out

    t = Probe(backend, split_from, pieces, piece_calls, len(piece_calls))
    t.fuse_bn_relu = fuse_bn_relu
    b = ShapeBinder(t, _Zeros())
    cache = {k: t.const(backend.empty(shape), shape) for k, shape in inputs.items()}
    build(t, b, cache)
    return level["peak"] - level["start"]


def trace_pieces(piece_build, piece_inputs, fuse_bn_relu=False):
    """The operator calls of the builder at the micro-tensors' batch size (graph.trace)."""
    from .workloads import ShapeBinder
    return graph.trace(piece_build, piece_inputs, lambda t: ShapeBinder(t, _Zeros()), fuse_bn_relu)


LINK_BYTES_PER_S = 57e9             # pinned host memory <-> HBM through DLArrayCopyFromTo, each way
HBM_BYTES_PER_S = 5e12              # what the streaming kernels that recompute a value sustain
SPLIT_ISSUE_MS_PER_OPERATOR = 0.04  # host time to issue one operator's forward and backward once more


def plan_split(ops, leaves_bytes, budget_bytes, build, inputs, piece_calls, pieces, lead=3, min_bytes=1 << 20,
               recompute=True, hold=1, fuse_bn_relu=False, always=False, split_from=None):
    """-> (TapePlan, the operators the plan refers to).  The plan over whole values is kept when it moves and
    recomputes nothing.  Otherwise (or with `always`) the end of the graph may run per micro-tensor: stretches
    that start 1, 2, 4, 8 ... operators before the loss, and at the first operator from which on nothing
    couples the samples of a batch, are planned as well, and the plan with the smallest estimated cost per step
    wins: bytes sent to the host and back at the link's rate, bytes recomputed at three passes over HBM, and, for
    a stretch, the host's time to issue its operators once more per extra micro-tensor (the kernels themselves do
    the same work on row ranges; SPLIT_ISSUE_MS_PER_OPERATOR was measured on the Transformer at batch 32, where a
    stretch over the whole graph in 4 pieces adds 73 ms to a 42 ms step).  plan.split_from / plan.pieces say what
    was chosen.  With `split_from` the stretch starts at that operator and nothing else is tried."""
    always = always or split_from is not None

    def cost(p, cut):
        ms = 2e3 * sum(cut[i].bytes for i in p.away) / LINK_BYTES_PER_S + 3e3 * sum(cut[i].bytes for i in p.redo) / HBM_BYTES_PER_S
        if p.split_from is not None:
            ms += (len(ops) - p.split_from) * (p.pieces - 1) * SPLIT_ISSUE_MS_PER_OPERATOR
        return ms

    best = None
    if not always:
        try:
            p = plan(ops, leaves_bytes, budget_bytes, lead, min_bytes, recompute, hold)
            if not p.away and not p.redo:
                return p, ops
            best = (cost(p, ops), p, ops)
        except ValueError:
            pass
    n = len(ops)
    assert len(piece_calls) == n, "the builder makes other calls at the micro-tensors' batch size"
    lowest = first_splittable(ops)
    starts, step = [], 1
    while n - 1 - step > lowest:
        starts.append(n - 1 - step)
        step *= 2
    starts.append(lowest)
    if split_from is not None:
        assert lowest <= split_from < n - 1, "a stretch run per micro-tensor starts at operator %d or later" % lowest
        starts = [split_from]
    last_error = None
    for s in starts:
        if s >= n - 1:
            continue
        cut = split_tail(ops, s, measure_tail(build, inputs, piece_calls, s, pieces, fuse_bn_relu))
        try:
            p = plan(cut, leaves_bytes, budget_bytes, lead, min_bytes, recompute, hold)
        except ValueError as e:
            last_error = e
            continue
        p.split_from, p.pieces = s, pieces
        if best is None or cost(p, cut) < best[0]:
            best = (cost(p, cut), p, cut)
    if best is None:
        raise last_error or ValueError("no operator of this graph can run per micro-tensor")
    return best[1], best[2]


class BudgetedTape(graph.MicroTape):
    """A Tape that executes `plan` (see the module description).  One instance per step; the streams
    and the pinned host buffers live in `state`, shared by the steps (BudgetedTape.make_state)."""

    class State(object):
        def __init__(self, ctx):
            self.ctx = ctx
            self.host_ctx = ndarray.cpu(0)
            self.out_stream = create_stream_handle(ctx)
            self.in_stream = create_stream_handle(ctx)
            self.host = {}           # operator -> pinned host array (kept across steps)
            self.peak_used = 0       # largest `used` figure of the device pool seen after an operator
            self.host_waits = 0

    @staticmethod
    def make_state(ctx):
        return BudgetedTape.State(ctx)

    def __init__(self, backend, tape_plan, ops, state, track_pool=False, piece_calls=None):
        if tape_plan.split_from is None:
            graph.MicroTape.__init__(self, backend)
        else:
            graph.MicroTape.__init__(self, backend, tape_plan.split_from, tape_plan.pieces, piece_calls, len(piece_calls))
        self.plan, self.ops, self.state = tape_plan, ops, state
        self.track_pool = track_pool
        n = len(ops)
        self.last_fwd, self.need = _needs(ops, tape_plan.redo)
        self.first = [max(r) if r else -1 for r in self.need]
        self.last = [min(r) if r else -1 for r in self.need]
        self.by_last_fwd = collections.defaultdict(list)
        for i in range(n):
            self.by_last_fwd[self.last_fwd[i]].append(i)
        self.by_last = collections.defaultdict(list)
        for i in range(n):
            if self.need[i]:
                self.by_last[self.last[i]].append(i)
        self.fetch_at = collections.defaultdict(list)
        for i in tape_plan.away:
            if self.need[i]:
                self.fetch_at[min(n - 1, self.first[i] + tape_plan.lead)].append(i)
        self.redo_at = collections.defaultdict(list)
        for i in tape_plan.redo:
            if self.need[i]:
                self.redo_at[self.first[i]].append(i)
        self.leaving = []            # (operator after which it is released, value, device array, event behind its
                                     #  last reader, copy-done event or None while the copy has not been issued)
        self.waiting_in = {}         # operator -> (event behind what was in flight when its memory was taken, array)
        self.arriving = {}           # operator -> copy-done event
        self.gone = set()            # values in host memory only
        self.recomputed = 0

    # ---- helpers
    def _compute_stream(self):
        return self.b.stream

    def _mark_compute(self):
        """An event at the current end of the compute stream."""
        ev = create_event_handle(self.state.ctx)
        ev.record(self._compute_stream())
        return ev

    def _reached(self, ev, wait):
        """True once `ev` has been reached; with `wait` the host waits for it (and that is counted)."""
        if ev.query():
            return True
        if wait:
            ev.sync()
            self.state.host_waits += 1
            return True
        return False

    def _inside_piece(self):
        self._note_pool()

    def _note_pool(self):
        if self.track_pool:
            from .gpu_memory_manager import pool_state
            self.state.peak_used = max(self.state.peak_used, pool_state().used)

    def _var(self, i):
        return self._nodes[i].out

    # A copy is issued once the compute stream has passed the point recorded when the copy was decided: the
    # last reader of a value that leaves, or everything that may still read the memory a returning value is
    # given.  The hooks look at those points as they pass (_poll) and issue what has become ready, so the
    # host waits only for a copy whose time has come: a value that is due for release, or one its reader needs.
    def _issue_out(self, entry, wait):
        due, i, arr, after, done = entry
        if done is None and self._reached(after, wait):
            host = self.state.host.get(i)
            if host is None or host.shape != arr.shape:
                host = self.state.host[i] = ndarray.empty(arr.shape, self.state.host_ctx)
            arr.copyto(host, self.state.out_stream)
            done = create_event_handle(self.state.ctx)
            done.record(self.state.out_stream)
        return (due, i, arr, after, done)

    def _issue_in(self, i, wait):
        pending = self.waiting_in.get(i)
        if pending is not None and self._reached(pending[0], wait):
            del self.waiting_in[i]
            self.state.host[i].copyto(pending[1], self.state.in_stream)
            ev = create_event_handle(self.state.ctx)
            ev.record(self.state.in_stream)
            self.arriving[i] = ev

    def _poll(self):
        self.leaving = [self._issue_out(e, False) for e in self.leaving]
        for i in list(self.waiting_in):
            self._issue_in(i, False)

    def _release_leaving(self, t=None):
        """Releases the values due after operator t (all of them without t) once their copies have left."""
        keep = []
        for entry in self.leaving:
            if t is not None and entry[0] > t:
                keep.append(entry)
                continue
            due, i, arr, after, done = self._issue_out(entry, True)
            self._reached(done, True)            # the copy has left the device
            del arr, entry
        self.leaving = keep

    # ---- hooks
    def _after_forward(self, node):
        t = node.index
        assert t < len(self.ops) and _bytes(node.out.shape) == self.ops[t].bytes, "the graph differs from the recorded one"
        self._note_pool()
        self._poll()
        self._release_leaving(t)
        n = len(self.ops)
        for i in self.by_last_fwd[t]:
            v = self._var(i)
            if not self.need[i] or i in self.plan.redo:
                if i != n - 1:
                    v.value = None       # nobody reads it again, or it will be computed again
            elif i in self.plan.away:
                # the operator that read it last has been issued: the copy out starts once it has run
                self.leaving.append((t + self.plan.hold, i, v.value, self._mark_compute(), None))
                v.value = None
                self.gone.add(i)

    def _fetch(self, i):
        v = self._var(i)
        # the memory is taken now (the plan counts it from here); the copy starts once nothing in flight can
        # still read memory the pool may have handed out for it
        arr = ndarray.empty(v.shape, self.state.ctx)
        self.waiting_in[i] = (self._mark_compute(), arr)
        v.value = arr
        self.gone.discard(i)

    def _ensure(self, i):
        """Value i is on the device and complete when this returns."""
        if i in self.gone:                     # (a value the plan fetches later than this reader needs it)
            self._fetch(i)
        self._issue_in(i, True)
        ev = self.arriving.pop(i, None)
        if ev is not None:
            self._reached(ev, True)
        if self._var(i).value is None and i in self.plan.redo:
            node = self._nodes[i]
            for u in node.inputs:
                if u.node >= 0:
                    self._ensure(u.node)
            node.out.value = node.redo()
            self.recomputed += 1

    def _before_backward(self, node):
        self._poll()
        for i in sorted(self.redo_at[node.index]):      # producers before consumers
            self._ensure(i)
        for s in node.saved:
            if s.node >= 0:
                self._ensure(s.node)

    def backward(self, loss):
        self._release_leaving()
        n = len(self.ops)
        assert len(self._nodes) == n, "the graph differs from the recorded one"
        for i in sorted(self.fetch_at[n - 1], key=lambda i: -self.first[i]):     # planned for the first operator
            if i in self.gone:
                self._fetch(i)
        graph.MicroTape.backward(self, loss)

    def _after_backward(self, node):
        # the sweep reaches operator j - 1 next: issue what the plan fetches there before its operators
        j = node.index
        self._note_pool()
        for i in self.by_last[j]:
            self._var(i).value = None
        if j > 0:
            for i in sorted(self.fetch_at[j - 1], key=lambda i: -self.first[i]):
                if i in self.gone:
                    self._fetch(i)
        self._poll()


class BudgetedRun(object):
    """Trains a graph step after step under a plan: `build(tape, binder, cache)` as for record();
    parameters come from `store` (workloads.ParamStore), inputs are numpy arrays uploaded once."""

    def __init__(self, build, inputs, store, budget_bytes, ctx=None, lead=3, track_pool=False, min_bytes=1 << 20,
                 recompute=True, hold=1, fuse_bn_relu=False, piece_build=None, pieces=1, split_always=False, split_from=None):
        """piece_build, pieces: the same builder for batch / pieces samples.  With them the planner may run the end
        of the graph per batch micro-tensor when whole values cannot meet the budget (plan_split), or does so
        in any case with `split_always`."""
        from . import stream, workloads
        self.ctx = ctx or ndarray.gpu(0)
        self.build = build
        self.fuse_bn_relu = fuse_bn_relu
        shapes = {k: tuple(np.shape(v)) for k, v in inputs.items()}
        self.ops, self.leaves_bytes = record(build, shapes, fuse_bn_relu)
        self.piece_calls = None
        if piece_build is not None and pieces > 1:
            assert all(sh[0] % pieces == 0 for sh in shapes.values()), "the batch must divide by the number of micro-tensors"
            self.piece_calls = trace_pieces(piece_build, {k: (sh[0] // pieces,) + sh[1:] for k, sh in shapes.items()}, fuse_bn_relu)
            self.plan, self.ops = plan_split(self.ops, self.leaves_bytes, budget_bytes, build, shapes, self.piece_calls, pieces,
                                             lead, min_bytes, recompute, hold, fuse_bn_relu, split_always, split_from)
        else:
            self.plan = plan(self.ops, self.leaves_bytes, budget_bytes, lead, min_bytes, recompute, hold)
        self._plan_args = (budget_bytes, min_bytes, recompute)
        self.stream = stream.create_stream_handle(self.ctx)
        self.backend = graph.GpuBackend(self.ctx, self.stream)
        self.state = BudgetedTape.make_state(self.ctx)
        self.track_pool = track_pool
        self.binder = None
        self.store = store
        self.inputs = inputs
        self.dev_inputs = None
        self._workloads = workloads

    def step(self, lr):
        """One forward + backward + SGD step; returns the loss Var (its value stays on the device)."""
        t = BudgetedTape(self.backend, self.plan, self.ops, self.state, self.track_pool, self.piece_calls)
        t.fuse_bn_relu = self.fuse_bn_relu
        if self.binder is None:
            self.binder = self._workloads.Binder(t, self.store)
            self.dev_inputs = {k: self.binder.input(v) for k, v in self.inputs.items()}
        else:
            self.binder.t, self.binder._n = t, 0
            for v in self.binder.vars.values():
                v.grad = None
        loss, _ = self.build(t, self.binder, self.dev_inputs)
        t.backward(loss)
        self.binder.sgd_step(lr)
        return loss

    def tune(self, lr, candidates=((3, 1), (30, 30), (60, 30), (100, 30), (200, 60), (400, 100)), steps=2):
        """Trains `steps` steps under each (lead, hold) schedule the budget admits and keeps the fastest.  Every
        plan computes the same bits, so these are ordinary training steps: only their speed differs (how far
        ahead of its reader a value starts coming back, how long a leaving value keeps its memory while its
        copy runs, and what else has to leave to make room for that).  The first step of a schedule is not
        timed (new pinned host buffers).  -> ((lead, hold), {(lead, hold): ms per step}), losses of the steps run."""
        import time
        budget_bytes, min_bytes, recompute = self._plan_args
        timings, plans, losses = {}, {}, []
        for lead, hold in candidates:
            try:
                plans[(lead, hold)] = plan(self.ops, self.leaves_bytes, budget_bytes, lead, min_bytes, recompute, hold)
            except ValueError:
                continue
            plans[(lead, hold)].split_from, plans[(lead, hold)].pieces = self.plan.split_from, self.plan.pieces
            self.plan = plans[(lead, hold)]
            losses.append(self.step(lr))
            self.sync()
            t0 = time.perf_counter()
            for _ in range(max(1, steps - 1)):
                losses.append(self.step(lr))
            self.sync()
            timings[(lead, hold)] = (time.perf_counter() - t0) / max(1, steps - 1) * 1e3
        if not timings:
            raise ValueError("no schedule fits the budget")
        best = min(timings, key=timings.get)
        self.plan = plans[best]
        return best, timings, losses

    def sync(self):
        self.backend.sync()


def max_batch(build_for, input_shapes_for, budget_bytes, planned=True, lead=3, limit=1 << 12, min_bytes=1 << 20,
              recompute=True, fuse_bn_relu=False):
    """Largest batch whose step fits `budget_bytes`: with `planned` the planner may send values to the
    host, without it the replayed peak of the plain schedule must fit.  build_for(batch) -> builder,
    input_shapes_for(batch) -> name -> shape.  The counterpart of the reference's batch-size sweeps per
    policy (examples/imagenet_resnet.py:139-154).  -> (batch, TapePlan) or (0, None)."""
    def fits(batch):
        ops, leaves = record(build_for(batch), input_shapes_for(batch), fuse_bn_relu)
        if any(op.bytes >= (1 << 33) for op in ops):      # tensors are limited to 2^31 elements
            return None
        try:
            p = plan(ops, leaves, budget_bytes if planned else None, lead, min_bytes, recompute)
        except ValueError:
            return None
        return p if p.peak_bytes <= budget_bytes else None

    best, best_plan, hi = 0, None, 1
    while hi <= limit:                 # double until it no longer fits
        p = fits(hi)
        if p is None:
            break
        best, best_plan = hi, p
        hi *= 2
    lo, hi = best, min(hi, limit + 1)
    while hi - lo > 1:
        mid = (lo + hi) // 2
        p = fits(mid)
        if p is None:
            hi = mid
        else:
            lo, best, best_plan = mid, mid, p
    return best, best_plan
