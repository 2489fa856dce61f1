"""Planner of the budgeted tape executor on recorded graphs (no GPU): the replay of the executor's
schedule and the greedy choice of what leaves the device."""
import numpy as np
import pytest

from tsplit_amd import tape_budget as tb, workloads


def _resnet(t, b, c):
    return workloads.resnet(t, b, c["x"], c["y"], blocks=(2, 2), base=8, classes=10)


def _inception(t, b, c):
    return workloads.inception_v4(t, b, c["x"], c["y"], n_a=1, n_b=1, n_c=1, div=8, classes=10)


SHAPES = {"resnet": (_resnet, {"x": (4, 3, 32, 32), "y": (4, 10)}),
          "inception": (_inception, {"x": (3, 3, 107, 107), "y": (3, 10)})}


@pytest.mark.parametrize("net", sorted(SHAPES))
def test_record_lists_every_operator_with_its_readers(net):
    build, shapes = SHAPES[net]
    ops, leaves = tb.record(build, shapes)
    assert leaves > sum(4 * int(np.prod(s)) for s in shapes.values())      # parameters are leaves too
    assert ops[-1].bytes == 4 and ops[-1].has_backward                      # the loss
    for t, op in enumerate(ops):
        assert all(i < t for i in op.inputs) and all(i <= t for i in op.saved)
        assert set(op.grad_inputs) <= set(op.inputs)
    # a convolution's backward reads its input, an addition's reads nothing
    last_fwd, bwd = tb._uses(ops)
    assert any(bwd[i] for i in range(len(ops))) and any(not bwd[i] for i in range(len(ops)))


@pytest.mark.parametrize("recompute", [False, True])
@pytest.mark.parametrize("net", sorted(SHAPES))
def test_plan_meets_the_budget_by_taking_idle_values_off_the_device(net, recompute):
    build, shapes = SHAPES[net]
    ops, leaves = tb.record(build, shapes)
    free_peak, at, idle = tb.replay(ops, leaves)
    assert free_peak > leaves and 0 <= at < 2 * len(ops)
    last_fwd, bwd = tb._uses(ops)
    for frac in (0.9, 0.7, 0.55):
        budget = leaves + int((free_peak - leaves) * frac)
        p = tb.plan(ops, leaves, budget, min_bytes=0, recompute=recompute)
        assert p.peak_bytes <= budget and p.free_peak_bytes == free_peak
        assert p.peak_bytes == tb.replay(ops, leaves, p.away, p.lead, p.redo)[0]
        last_fwd, need = tb._needs(ops, p.redo)
        assert all(need[i] for i in p.away | p.redo)     # only values that are read again are worth taking off
        assert not (p.away & p.redo) and all(ops[i].cheap for i in p.redo)
        assert recompute or not p.redo
    if recompute:
        # what is computed again is never sent over the link as well, and less travels than without
        moved = sum(ops[i].bytes for i in p.away)
        q = tb.plan(ops, leaves, budget, min_bytes=0, recompute=False)
        assert moved < sum(ops[i].bytes for i in q.away)
    none = tb.plan(ops, leaves, None)
    assert none.away == frozenset() and none.redo == frozenset()
    with pytest.raises(ValueError):
        tb.plan(ops, leaves, leaves + 1, min_bytes=0)


def test_a_recomputed_value_keeps_its_inputs_until_it_has_been_rebuilt():
    """Dropping a Relu output makes the BatchNorm output before it needed at the Relu output's first
    backward reader, which is earlier in the sweep than the BatchNorm output's own reader."""
    build, shapes = SHAPES["resnet"]
    ops, leaves = tb.record(build, shapes)
    last_fwd, bwd = tb._uses(ops)
    # a cheap operator whose single input is an operator output that its own backward reads (Relu after BatchNorm)
    i = next(k for k, op in enumerate(ops) if op.cheap and len(op.inputs) == 1 and op.inputs[0] >= 0 and bwd[k]
             and ops[op.inputs[0]].cheap)
    u = ops[i].inputs[0]
    _, need = tb._needs(ops, {i})
    assert max(need[u]) == max(bwd[i]) >= max(bwd[u])
    _, need2 = tb._needs(ops, {i, u})           # chains: the convolution output before the BatchNorm as well
    assert max(need2[ops[u].inputs[0]]) == max(bwd[i])


def test_sending_a_value_away_frees_it_between_its_uses():
    build, shapes = SHAPES["resnet"]
    ops, leaves = tb.record(build, shapes)
    last_fwd, bwd = tb._uses(ops)
    # the largest value that the backward sweep reads again
    i = max((op.bytes, k) for k, op in enumerate(ops) if bwd[k])[1]
    base = tb.replay(ops, leaves)[0]
    assert tb.replay(ops, leaves, {i})[0] <= base
    j = max((op.bytes, k) for k, op in enumerate(ops) if bwd[k] and op.cheap)[1]
    assert tb.replay(ops, leaves, (), 3, {j})[0] <= base


def test_holding_and_fetching_ahead_cost_memory_that_the_plan_makes_room_for():
    """A leaving value that keeps its memory for `hold` operators and a returning one that takes its memory
    `lead` operators early raise the replayed peak of a given choice; the planner answers by sending more
    away, still within the budget; a schedule that holds everything to the end of the sweep saves nothing."""
    build, shapes = SHAPES["resnet"]
    ops, leaves = tb.record(build, shapes)
    free_peak = tb.replay(ops, leaves)[0]
    budget = leaves + int((free_peak - leaves) * 0.6)
    tight = tb.plan(ops, leaves, budget, lead=3, min_bytes=0, recompute=False, hold=1)
    assert tight.away and tight.peak_bytes <= budget and (tight.lead, tight.hold) == (3, 1)
    # the same choice replayed under lazier schedules: never a lower peak
    peaks = [tb.replay(ops, leaves, tight.away, lead, (), hold)[0] for lead, hold in ((3, 1), (3, 4), (8, 4), (20, 12))]
    assert peaks[0] == tight.peak_bytes and all(b >= a for a, b in zip(peaks, peaks[1:]))
    lazy = tb.plan(ops, leaves, budget, lead=8, min_bytes=0, recompute=False, hold=4)
    assert lazy.peak_bytes <= budget and len(lazy.away) >= len(tight.away) and (lazy.lead, lazy.hold) == (8, 4)
    assert tb.replay(ops, leaves, lazy.away, 8, (), 4)[0] == lazy.peak_bytes
    n = len(ops)
    assert tb.replay(ops, leaves, tight.away, n, (), n)[0] == free_peak
    with pytest.raises(ValueError):
        tb.plan(ops, leaves, budget, lead=n, min_bytes=0, recompute=False, hold=n)


def test_max_batch_grows_with_the_budget_and_with_planning():
    def build_for(batch):
        return _resnet

    def shapes_for(batch):
        return {"x": (batch, 3, 32, 32), "y": (batch, 10)}
    budget = 8 << 20
    plain, _ = tb.max_batch(build_for, shapes_for, budget, planned=False, limit=512)
    planned, p = tb.max_batch(build_for, shapes_for, budget, planned=True, limit=512, min_bytes=0)
    assert 0 < plain < planned and p.peak_bytes <= budget
    more, _ = tb.max_batch(build_for, shapes_for, 2 * budget, planned=False, limit=512)
    assert more > plain
