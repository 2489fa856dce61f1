"""Host-side checks of the memory planner: the allocation replay, the greedy choice and the
layer-list fusion.  No GPU work."""
import numpy as np
import pytest

from tsplit_amd import planner, trainer

SMALL = [("conv", "c1", 3, 8, 3, 1, 1), ("bn", "c1_bn", 8), ("relu",), ("conv", "c2", 8, 8, 3, 1, 1), ("bn", "c2_bn", 8),
         ("relu",), ("maxpool", 2, 0, 2), ("flatten",), ("fc", "f1", 8 * 8 * 8, 10)]
IN = (4, 3, 16, 16)


def test_fuse_spec_merges_bn_relu_pairs_only():
    f = planner.fuse_spec(SMALL)
    assert [l[0] for l in f] == ["conv", "bnrelu", "conv", "bnrelu", "maxpool", "flatten", "fc"]
    assert f[1] == ("bnrelu", "c1_bn", 8)
    assert planner.fuse_spec([("bn", "x", 4), ("maxpool", 2, 0, 2), ("relu",)]) == [("bn", "x", 4), ("maxpool", 2, 0, 2), ("relu",)]
    assert planner.layer_shapes(f, IN)[-1] == (4, 10)


def test_fuse_spec_takes_the_pooling_behind_a_pair_where_the_planes_are_even():
    f = planner.fuse_spec(SMALL, pool=True, input_shape=IN)
    assert [l[0] for l in f] == ["conv", "bnrelu", "conv", "bnrelupool", "flatten", "fc"]
    assert f[3] == ("bnrelupool", "c2_bn", 8)
    assert planner.layer_shapes(f, IN)[4] == (4, 8, 8, 8) and planner.layer_shapes(f, IN)[-1] == (4, 10)
    # odd planes, other windows or a pooling that does not follow directly stay as they are
    odd = planner.fuse_spec(SMALL, pool=True, input_shape=(4, 3, 15, 15))
    assert [l[0] for l in odd] == ["conv", "bnrelu", "conv", "bnrelu", "maxpool", "flatten", "fc"]
    other = [("bn", "x", 4), ("relu",), ("maxpool", 3, 1, 2)]
    assert [l[0] for l in planner.fuse_spec(other, pool=True, input_shape=(2, 4, 8, 8))] == ["bnrelu", "maxpool"]
    # the activation in front of the pooling never exists: VGG-16 at batch 64 holds 1.57 GB less
    spec = trainer.vgg16_spec(1000, 224)
    shape = (64, 3, 224, 224)
    pairs = planner.plan_memory(planner.fuse_spec(spec), shape, None, 0)
    ends = planner.plan_memory(planner.fuse_spec(spec, pool=True, input_shape=shape), shape, None, 0)
    shapes = planner.layer_shapes(spec, shape)
    pre_pool = sum(planner.tensor_bytes(shapes)[i] for i, l in enumerate(spec) if l[0] == "maxpool")
    assert pairs.peak_bytes - ends.peak_bytes >= pre_pool > 1.5e9


def test_simulate_without_swapping_holds_every_activation_at_the_turn():
    shapes = planner.layer_shapes(SMALL, IN)
    size = planner.tensor_bytes(shapes)
    peak, events = planner.simulate(SMALL, shapes, (), fixed_bytes=1000)
    # last backward layer (fc): all activations but the logits (only their gradient is read from here on)
    # + logits gradient + the fc input gradient
    turn = [e for e in events if e[0] == "bwd" and e[1] == len(SMALL) - 1][0]
    assert turn[2] == 1000 + sum(size[:-1]) + size[-1] + size[-2]
    # max pooling reads its own output in the backward pass: still resident then
    pool = [i for i, l in enumerate(SMALL) if l[0] == "maxpool"][0]
    at_pool = [e for e in events if e[0] == "bwd" and e[1] == pool][0]
    assert pool + 1 in at_pool[3]
    conv = [i for i, l in enumerate(SMALL) if l[0] == "conv"][-1]
    assert conv + 1 not in [e for e in events if e[0] == "bwd" and e[1] == conv][0][3]
    assert peak == max(e[2] for e in events) >= turn[2]
    # forward residency grows by one tensor per layer
    fwd = [e[2] for e in events if e[0] == "fwd"]
    assert fwd == [1000 + sum(size[:i + 2]) for i in range(len(SMALL))]


def test_swapping_lowers_the_peak_and_in_place_gradients_cost_nothing():
    shapes = planner.layer_shapes(SMALL, IN)
    size = planner.tensor_bytes(shapes)
    base, _ = planner.simulate(SMALL, shapes, ())
    less, events = planner.simulate(SMALL, shapes, (1, 2, 3), prefetch=1)
    assert less < base
    # while layer 5 runs backward (Relu, in place) tensors 1..3 are away, its own output (6) is
    # already released and one gradient is live
    e5 = [e for e in events if e[0] == "bwd" and e[1] == 5][0]
    assert not ({1, 2, 3, 6} & set(e5[3])) and {4, 5} <= set(e5[3])
    assert e5[2] == sum(size[j] for j in e5[3]) + size[6]
    # one layer ahead: tensor 3 is back while layer 4 runs backward
    e4 = [e for e in events if e[0] == "bwd" and e[1] == 4][0]
    assert 3 in e4[3] and 2 not in e4[3]


def test_plan_meets_budgets_and_swaps_more_as_they_shrink():
    fixed = 4096
    free = planner.plan_memory(SMALL, IN, None, fixed)
    assert not free.swap and not free.split
    shapes = planner.layer_shapes(SMALL, IN)
    floor, _ = planner.simulate(SMALL, shapes, range(1, len(SMALL)), fixed)     # everything that may leave has left
    assert floor < free.peak_bytes
    prev = set()
    for frac in (0.9, 0.5, 0.0):
        budget = int(floor + frac * (free.peak_bytes - floor))
        p = planner.plan_memory(SMALL, IN, budget, fixed, piece_bytes=2048)
        assert p.peak_bytes <= budget
        assert 0 not in p.swap and len(SMALL) not in p.swap
        assert len(p.swap) >= len(prev)
        prev = set(p.swap)
        for li, k in p.split.items():
            assert SMALL[li][0] == "conv" and li in p.swap and 1 < k <= IN[0]
    d = p.describe()
    assert d["swap"] == sorted(p.swap) and d["budget_GiB"] == budget / planner.GiB


def test_plan_raises_when_nothing_more_can_leave():
    with pytest.raises(ValueError, match="cannot be met"):
        planner.plan_memory(SMALL, IN, 1024, 0)


def test_vgg16_batch64_numbers():
    """The unplanned peak of VGG-16 b64: 3 x 527.8 MiB of parameter-sized arrays plus 39 conv-block
    tensors, pools, FC activations, and two gradients at the widest point."""
    spec = trainer.vgg16_spec(1000, 224)
    shapes = planner.layer_shapes(spec, (64, 3, 224, 224))
    size = planner.tensor_bytes(shapes)
    conv_out = sum(size[i + 1] for i, l in enumerate(spec) if l[0] == "conv")
    assert conv_out == 4 * 867041280                     # 867.0 M conv-output elements per step
    fused = planner.fuse_spec(spec)
    p_plain = planner.plan_memory(spec, (64, 3, 224, 224), None, 0)
    p_fused = planner.plan_memory(fused, (64, 3, 224, 224), None, 0)
    assert p_plain.peak_bytes - p_fused.peak_bytes == conv_out    # the BatchNorm outputs never exist
    tight = planner.plan_memory(fused, (64, 3, 224, 224), 6 << 30, 1660 << 20)
    assert tight.peak_bytes <= 6 << 30 and tight.swap


def test_copy_ins_start_early_where_the_budget_allows_and_keep_the_order_of_need():
    spec = planner.fuse_spec(trainer.vgg16_spec(1000, 224))
    shape = (64, 3, 224, 224)
    p = planner.plan_memory(spec, shape, 7 << 30, 1660 << 20)
    assert p.swap and set(p.issue_at) == set(p.swap)
    order = sorted(p.swap, reverse=True)
    for j in order:
        assert p.issue_at[j] >= min(len(spec) - 1, j + p.prefetch)           # never later than the minimum lead
    assert all(p.issue_at[a] >= p.issue_at[b] for a, b in zip(order, order[1:]))   # needed first, issued first
    assert any(p.issue_at[j] > j + p.prefetch for j in order)                      # some did move
    shapes = planner.layer_shapes(spec, shape)
    peak, _ = planner.simulate(spec, shapes, p.swap, p.fixed_bytes, p.prefetch, p.issue_at)
    assert peak == p.peak_bytes <= 7 << 30
    cost = planner.CostModel()
    assert planner.step_ms(spec, shapes, p.swap, cost, p.prefetch, p.issue_at) <= \
        planner.step_ms(spec, shapes, p.swap, cost, p.prefetch)


def test_max_batch_grows_with_the_budget_and_with_planning():
    """The largest batch under a budget: never smaller with a bigger budget, larger with planning than
    with everything resident, its plan replays within the budget, and one image more does not fit."""
    from tsplit_amd import planner, trainer
    from tsplit_amd.planned_trainer import fixed_bytes, make_plan, max_batch
    spec = trainer.vgg16_spec(10, 32)
    opt = ("momentum", 0.01, 0.9)
    image = (3, 32, 32)
    last = (0, 0)
    for mib in (600, 800, 1200):
        budget = mib << 20
        resident, _ = max_batch(spec, image, 10, budget, opt, swap=False)
        planned, plan = max_batch(spec, image, 10, budget, opt, swap=True)
        assert planned > resident > 0
        assert resident >= last[0] and planned >= last[1]
        last = (resident, planned)
        shapes = planner.layer_shapes(spec, (planned,) + image)
        peak, _ = planner.simulate(spec, shapes, plan.swap, fixed_bytes(spec, (planned,) + image, 10, opt, tuple(plan.split)))
        assert peak <= budget
        with pytest.raises(ValueError):
            make_plan(spec, (planned + 1,) + image, 10, budget, opt)
        free = make_plan(spec, (resident + 1,) + image, 10, None, opt)
        assert free.peak_bytes > budget


def test_recomputation_replay_and_choice():
    """Dropped tensors leave after their forward use and are back, with the tensor they are computed
    from, when their layer's backward runs; chains (Relu output from BatchNorm output from the kept
    convolution output) replay in order; a tensor something is recomputed from is never swapped; the
    estimated step never gets slower by allowing recomputation."""
    from tsplit_amd import planner, trainer
    from tsplit_amd.planned_trainer import fixed_bytes, make_plan
    spec = trainer.vgg16_spec(10, 32)
    shape = (64, 3, 32, 32)
    opt = ("momentum", 0.01, 0.9)
    shapes = planner.layer_shapes(spec, shape)
    size = planner.tensor_bytes(shapes)
    # hand-made: drop BN output (tensor 2) and Relu output (tensor 3) of the first block
    peak0, _ = planner.simulate(spec, shapes)
    peak, events = planner.simulate(spec, shapes, recompute=(2, 3))
    assert peak <= peak0
    fwd = {li: res for ph, li, _, res, _ in events if ph == "fwd"}
    assert 2 in fwd[2] and 2 not in fwd[3] and 3 in fwd[3] and 3 not in fwd[4]
    redone = [(li, res) for ph, li, _, res, _ in events if ph == "re"]
    assert [li for li, _ in redone] == [2, 3]                  # the chain is rebuilt front to back
    assert {1, 2} <= redone[0][1] and {2, 3} <= redone[1][1]
    bwd = {li: res for ph, li, _, res, _ in events if ph == "bwd"}
    assert 3 in bwd[3] and 4 not in bwd[3] and 2 in bwd[2] and 3 not in bwd[2] and 1 in bwd[1] and 2 not in bwd[1]
    free = make_plan(spec, shape, 10, None, opt)
    floor = planner.simulate(spec, shapes, range(1, len(spec)), free.fixed_bytes)[0]
    for frac in (0.7, 0.4, 0.15):
        budget = int(floor + frac * (free.peak_bytes - floor))
        both = make_plan(spec, shape, 10, budget, opt, allow_recompute=True)
        swap_only = make_plan(spec, shape, 10, budget, opt)
        assert both.recompute and both.peak_bytes <= budget
        assert both.est_step_ms <= swap_only.est_step_ms + 1e-9
        for j in both.recompute:
            assert spec[j - 1][0] in planner.CHEAP_TO_REDO
            k = j - 1
            while k in both.recompute:
                k -= 1
            assert k not in both.swap
        again = planner.simulate(spec, shapes, both.swap, fixed_bytes(spec, shape, 10, opt, tuple(both.split)),
                                 issue_at=both.issue_at, recompute=both.recompute)[0]
        assert again == both.peak_bytes


def test_step_estimate_waits_only_where_the_executor_does():
    """One swapped tensor, worked by hand: the copy-out starts with its consumer and holds nothing up
    before the turn; the copy-in is issued `prefetch` layers ahead and the consumer's backward waits for
    it; a budget that leaves no room makes an allocation wait for the copy-out instead."""
    shapes = planner.layer_shapes(SMALL, IN)
    size = planner.tensor_bytes(shapes)
    cost = planner.CostModel(link_gbs=0.05, host_wait_ms=0.0)        # slow link: the copies outlast the layers
    f, b = planner.layer_times(SMALL, shapes, cost)
    L, c = len(SMALL), cost.copy_ms(size[1])
    free = planner.step_ms(SMALL, shapes, (), cost)
    assert free == pytest.approx(sum(f) + sum(b))
    t = max(sum(f), f[0] + c)                                          # the turn waits for the copy-out
    issue = min(L - 1, 1 + 3)
    t += sum(b[issue + 1:])                                            # backward of the layers behind the issue point
    arrival = t + c
    t += sum(b[2:issue + 1])
    t = max(t, arrival) + b[1] + b[0]
    assert planner.step_ms(SMALL, shapes, (1,), cost) == pytest.approx(t)
    # each host-side wait of a swap (one on the way out, one on the way in) is charged to the compute stream
    quick = planner.CostModel(link_gbs=1e6, host_wait_ms=0.5)
    assert planner.step_ms(SMALL, shapes, (1,), quick) == pytest.approx(planner.step_ms(SMALL, shapes, (), quick) + 1.0, abs=1e-3)
    # with room for everything the budget changes nothing; at the replayed peak of this plan the first
    # allocation that does not fit beside tensor 1 waits for it to have left, and the rest of the forward
    # pass runs after the copy instead of under it
    roomy, _ = planner.simulate(SMALL, shapes, ())
    assert planner.step_ms(SMALL, shapes, (1,), cost, budget_bytes=roomy) == pytest.approx(t)
    tight, _ = planner.simulate(SMALL, shapes, (1,))
    assert tight < roomy and f[0] + c > sum(f)
    held, first_wait = size[0], None
    for li in range(L):
        held += size[li + 1]
        if held > tight:
            first_wait = li
            break
    assert first_wait is not None and first_wait >= 2
    assert planner.step_ms(SMALL, shapes, (1,), cost, budget_bytes=tight) == pytest.approx(t + sum(f[first_wait:]))
