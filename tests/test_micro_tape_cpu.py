"""The end of a graph run per batch micro-tensor (tsplit_amd.graph.MicroTape) against the same graph
on the plain tape, both on the numpy oracle backend (no GPU): the stretch's forward and backward run
piece by piece on zero-copy row ranges of the outside values, and the loss and every parameter gradient
must come out as from the whole batch - for a Transformer (everything may be split: stretches that
start at the logits, in the middle of the decoder, and at the very first operator) and for a ResNet,
whose BatchNorm layers couple the samples, so only what follows the last one may be split.  Then the
planner's side: what the counting backend says a stretch holds, and a budget no plan over whole values
can meet but a plan with a micro-tensor stretch can."""
import numpy as np
import pytest

from oracle_backend import OracleBackend
from tsplit_amd import graph, tape_budget as tb, workloads


def _transformer(batch, vocab=50):
    cfg = workloads.TransformerConfig(batch=batch, len1=10, len2=8, d_model=32, heads=4, d_ff=64, blocks=1, vocab=vocab,
                                      mask_value=-1.0, embed_std=0.05, pos_amplitude=0.2)
    return lambda t, b, c: workloads.transformer(t, b, cfg, c["xs"], c["yi"], c["yo"])


def _transformer_inputs(rng, batch):
    ids = lambda n: rng.randint(0, 50, size=(batch, n)).astype(np.float32)
    xs, yi, yo = ids(10), ids(8), ids(8)
    xs[:, -2:] = 0
    yi[:, -1] = 0
    return {"xs": xs, "yi": yi, "yo": yo}


def _resnet(batch):
    return lambda t, b, c: workloads.resnet(t, b, c["x"], c["y"], blocks=(1, 1), base=4, classes=10)


def _resnet_inputs(rng, batch):
    y = np.zeros((batch, 10), np.float32)
    y[np.arange(batch), rng.randint(0, 10, batch)] = 1
    return {"x": rng.normal(size=(batch, 3, 32, 32)).astype(np.float32), "y": y}


def _run(tape, build, inputs, seed):
    b = workloads.Binder(tape, workloads.ParamStore(seed))
    cache = {k: b.input(v) for k, v in inputs.items()}
    loss, _ = build(tape, b, cache)
    tape.backward(loss)
    return float(np.asarray(loss.value)[0]), b.grads()


def _piece_calls(build_for, inputs, pieces):
    shapes = {k: (v.shape[0] // pieces,) + v.shape[1:] for k, v in inputs.items()}
    return tb.trace_pieces(build_for(inputs["xs" if "xs" in inputs else "x"].shape[0] // pieces), shapes)


@pytest.mark.parametrize("pieces,start", [(2, "logits"), (4, "logits"), (2, "middle"), (4, "first"), (1, "first")])
def test_transformer_end_per_micro_tensor_equals_the_whole_batch(pieces, start, rng):
    batch = 4
    inputs = _transformer_inputs(rng, batch)
    want_loss, want = _run(graph.Tape(OracleBackend()), _transformer(batch), inputs, 7)
    calls = _piece_calls(_transformer, inputs, pieces)
    n = len(calls)
    names = [c[0] for c in calls]
    split_from = {"logits": max(i for i, nm in enumerate(names) if nm == "matmul") - 1, "middle": n // 2, "first": 0}[start]
    t = graph.MicroTape(OracleBackend(), split_from, pieces, calls, n)
    got_loss, got = _run(t, _transformer(batch), inputs, 7)
    assert abs(got_loss - want_loss) <= 1e-6 * abs(want_loss)
    assert set(got) == set(want)
    for k in want:
        scale = max(np.max(np.abs(want[k])), 1e-30)
        assert np.max(np.abs(got[k] - want[k])) <= 2e-6 * scale, k


def test_resnet_tail_per_micro_tensor_and_batchnorm_is_refused(rng):
    batch, pieces = 4, 2
    inputs = _resnet_inputs(rng, batch)
    want_loss, want = _run(graph.Tape(OracleBackend()), _resnet(batch), inputs, 3)
    ops, _ = tb.record(_resnet(batch), {k: v.shape for k, v in inputs.items()})
    calls = _piece_calls(_resnet, inputs, pieces)
    lowest = tb.first_splittable(ops)
    assert 0 < lowest < len(ops) - 1 and ops[lowest - 1].name in graph.COUPLES_SAMPLES
    t = graph.MicroTape(OracleBackend(), lowest, pieces, calls, len(calls))
    got_loss, got = _run(t, _resnet(batch), inputs, 3)
    assert abs(got_loss - want_loss) <= 1e-6 * abs(want_loss)
    for k in want:
        assert np.max(np.abs(got[k] - want[k])) <= 2e-6 * max(np.max(np.abs(want[k])), 1e-30), k
    with pytest.raises(AssertionError):
        graph.MicroTape(OracleBackend(), lowest - 1, pieces, calls, len(calls))      # a BatchNorm inside the stretch


def test_planner_takes_a_micro_tensor_stretch_when_whole_values_cannot_meet_the_budget():
    batch, pieces, vocab = 8, 4, 8000          # a vocabulary this wide puts the peak at the logits, as at full size
    build = _transformer(batch, vocab)
    shapes = {"xs": (batch, 10), "yi": (batch, 8), "yo": (batch, 8)}
    ops, leaves = tb.record(build, shapes)
    calls = tb.trace_pieces(_transformer(batch // pieces, vocab), {k: (batch // pieces,) + s[1:] for k, s in shapes.items()})
    assert [c[0] for c in calls] == [op.name for op in ops]
    # the floor of plans over whole values: the smallest budget plan() accepts
    lo, hi = leaves, tb.replay(ops, leaves)[0]
    while hi - lo > 64:
        mid = (lo + hi) // 2
        try:
            tb.plan(ops, leaves, mid, min_bytes=0)
            hi = mid
        except ValueError:
            lo = mid
    floor = hi
    budget = leaves + int(0.6 * (floor - leaves))
    with pytest.raises(ValueError):
        tb.plan(ops, leaves, budget, min_bytes=0)
    p, cut = tb.plan_split(ops, leaves, budget, build, shapes, calls, pieces, min_bytes=0)
    assert p.split_from is not None and p.pieces == pieces and len(cut) == p.split_from + 1
    assert p.peak_bytes <= budget and cut[-1].name == "micro_tensor_tail" and cut[-1].transient > 0
    # a budget whole values can meet is met without a stretch
    q, same = tb.plan_split(ops, leaves, hi * 2, build, shapes, calls, pieces, min_bytes=0)
    assert q.split_from is None and same is ops
    # what a stretch holds shrinks with the number of pieces
    s = p.split_from
    held = {k: tb.measure_tail(build, shapes, tb.trace_pieces(_transformer(batch // k, vocab),
                                                              {n: (batch // k,) + sh[1:] for n, sh in shapes.items()}), s, k)
            for k in (1, 2, 4)}
    assert held[4] < held[2] < held[1]
