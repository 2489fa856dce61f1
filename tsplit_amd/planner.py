"""Memory planner for the sequential-net trainer: which saved activations leave the device
between their forward and backward use, and in how many batch micro-tensors the layers around
them run, so that a training step fits a device-memory budget.

The reference ships the primitives for this (batch micro-tensor views, DLArrayReuseAlloc, the
swap copies and events: src/common/c_runtime_api.cc:164-271, python/athena/ndarray.py:221-243,
351-409) and the tensor-granularity policies built on them (python/athena/gpu_ops/
vdnnExecutor.py:202-330), but not the planner that chooses splits; this module is that planner
for the layer lists of `tsplit_amd.trainer`.

Model.  Tensor j is the input of layer j (tensor 0 is the batch, tensor L the logits).  Every
tensor is needed again in the backward sweep (by the layer that consumed it, and a max-pool's
output also by the pool itself).  A BatchNorm directly followed by a Relu may be merged into one
"bnrelu" layer (`fuse_spec`), which runs on the fused entry points and never materialises the
BatchNorm output; with a 2x2 / stride 2 max pooling behind the pair the three may be merged into one
"bnrelupool" layer, which never materialises the activation in front of the pooling either and does not
need its own output in the backward sweep.  The executor (`tsplit_amd.planned_trainer`) follows this
schedule, which `simulate` replays byte for byte:

  forward  of layer i : allocate tensor i+1, run; then a swapped tensor i starts leaving
                        (it left the compute stream's hands) and is released once its copy is done
  backward of layer i : tensor i must be resident (a swapped one was re-allocated and its
                        copy-in issued at the start of an earlier layer's backward: at least
                        `prefetch` layers ahead, earlier where the budget has room, always in
                        the order of need);
                        allocate the input gradient unless the layer writes it in place
                        (Relu, BatchNorm: elementwise in the gradient); run; release tensor
                        i+1 and the output gradient

Choice.  Greedy: while the replayed peak exceeds the budget, take the moment of the peak and,
among the tensors resident but idle then, remove the one that adds the least estimated step
time per byte it frees - by swapping it, or (if allowed, and a cheap layer produced it) by
dropping it and computing it again in the backward sweep.  The estimate (`step_ms`) walks the
same schedule with a cost model: layer times from measured rates, one copy at a time per link
direction, and waits where the executor waits (an allocation that does not fit the budget
without an outstanding release, the turn, a layer whose copy-in has not arrived, the host-side
event waits of a swap) - so a tensor whose transfer hides behind a long convolution is cheap,
and a run of neighbouring small tensors that would queue on the link is not.  Layers
whose input is swapped run in micro-tensors of at most `piece_bytes`, so that a backward
micro-op starts as soon as its own piece has arrived.
"""
import collections
import math

import numpy as np

GiB = float(1 << 30)


class CostModel(object):
    """Rates measured on one MI355X with this library (fp32): contractions (for wide 3x3 layers the
    rate of the direct algorithm's FLOP count under the Winograd routine), streaming
    kernels on the bytes they move, the pinned-host link each way, and what one host-side
    event wait costs the compute stream (the host has to catch up with its launches afterwards;
    a swapped tensor brings one such wait on the way out and one on the way in)."""

    def __init__(self, conv_tflops=110.0, conv_tflops_narrow=90.0, matmul_tflops=45.0, stream_gbs=6000.0,
                 link_gbs=55.0, host_wait_ms=0.2, thin_gbs=2900.0):
        self.host_wait_ms = host_wait_ms
        self.conv_tflops = conv_tflops
        self.conv_tflops_narrow = conv_tflops_narrow
        self.matmul_tflops = matmul_tflops
        self.stream_gbs = stream_gbs
        self.link_gbs = link_gbs
        self.thin_gbs = thin_gbs

    @staticmethod
    def winograd_tflops(cin, cout, plane):
        """Rate of the direct algorithm's FLOP count of a 3x3 / stride 1 / pad 1 layer under the Winograd routine
        (all three passes together), as measured layer by layer on the VGG-16 shapes: the transforms' share
        falls and the GEMMs' depth grows with the channel count; the 14 x 14 planes leave a sparse last round."""
        lo, hi = min(cin, cout), max(cin, cout)
        if lo < 128:
            return 262.0 if hi < 128 else 237.0      # one kernel per pass
        if lo < 256:
            return 291.0 if hi < 256 else 302.0      # forward / data gradient one kernel; filter gradient too up to 128
        if lo < 512:
            return 332.0 if hi < 512 else 313.0
        return 368.0 if plane >= 28 else 235.0

    def copy_ms(self, nbytes):
        return nbytes / (self.link_gbs * 1e9) * 1e3

    def layer_ms(self, layer, in_shape, out_shape, backward, first=False):
        """Estimated time of one layer's forward (or backward) sweep."""
        n_in, n_out = float(np.prod(in_shape)), float(np.prod(out_shape))
        kind = layer[0]
        if kind == "conv":
            _, _, cin, cout, k, pad, stride = layer
            flop = 2.0 * n_out * cin * k * k
            passes = (1 if first else 2) if backward else 1
            if cin * k * k <= 32:      # a first layer on 3 channels: bound by writing (reading) the wide side
                return passes * 4.0 * (n_in + n_out) / (self.thin_gbs * 1e9) * 1e3
            rate = self.conv_tflops if min(cin, cout) > 64 else self.conv_tflops_narrow
            if (k, pad, stride) == (3, 1, 1) and min(cin, cout) >= 64:
                rate = self.winograd_tflops(cin, cout, out_shape[2])     # wide 3x3 layers run through the Winograd routine
            return passes * flop / (rate * 1e12) * 1e3
        if kind == "fc":
            flop = 2.0 * in_shape[0] * layer[2] * layer[3]
            return (2 if backward and not first else 1) * flop / (self.matmul_tflops * 1e12) * 1e3
        moved = {"bn": (20.0 if backward else 12.0) * n_in, "relu": (12.0 if backward else 8.0) * n_in,
                 "bnrelu": (20.0 if backward else 12.0) * n_in,
                 "bnrelupool": (14.0 if backward else 9.0) * n_in,
                 "maxpool": 4.0 * ((2 * n_in + n_out) if backward else (n_in + n_out)),
                 "flatten": 0.0}[kind]
        return moved / (self.stream_gbs * 1e9) * 1e3


IN_PLACE_BACKWARD = ("relu", "bn", "bnrelu")   # the input gradient may overwrite the output gradient
NEEDS_OUTPUT_BACKWARD = ("maxpool",)           # CuDNN_DLGpuMax_Pooling2d_gradient takes y as well as x
# layers whose output is cheap to compute again from their input (two or three passes over HBM):
# such an output may be dropped after its forward use and recomputed when the backward sweep needs it
CHEAP_TO_REDO = ("relu", "bn", "bnrelu", "bnrelupool")


class MemoryPlan(object):
    def __init__(self, swap, split, peak_bytes, est_step_ms, est_free_step_ms, fixed_bytes, budget_bytes, prefetch,
                 issue_at=None, recompute=()):
        self.swap = frozenset(swap)          # tensor indices that leave the device after their forward use
        # tensor indices dropped after their forward use and computed again, from the tensor before,
        # when the backward sweep reaches them
        self.recompute = frozenset(recompute)
        self.split = dict(split)             # layer index -> batch micro-tensors
        self.prefetch = prefetch             # least lead, in layers, of a copy-in over the backward sweep
        # tensor -> backward layer at whose start its copy-in is issued
        self.issue_at = dict(issue_at) if issue_at is not None else {j: j + prefetch for j in self.swap}
        self.peak_bytes = peak_bytes
        self.est_step_ms = est_step_ms             # cost-model step time with this plan ...
        self.est_free_step_ms = est_free_step_ms   # ... and with nothing swapped
        self.fixed_bytes = fixed_bytes
        self.budget_bytes = budget_bytes

    def describe(self):
        return {"swap": sorted(self.swap), "recompute": sorted(self.recompute), "split": {int(k): int(v) for k, v in sorted(self.split.items())},
                "prefetch": self.prefetch, "issue_at": {int(k): int(v) for k, v in sorted(self.issue_at.items())},
                "peak_GiB": self.peak_bytes / GiB, "est_step_ms": self.est_step_ms,
                "est_free_step_ms": self.est_free_step_ms,
                "fixed_GiB": self.fixed_bytes / GiB,
                "budget_GiB": None if self.budget_bytes is None else self.budget_bytes / GiB}


def fuse_spec(spec, pool=False, input_shape=None):
    """("bn", name, C), ("relu",) -> ("bnrelu", name, C); with `pool` (and the net's input shape, to know the
    planes) a pair followed by ("maxpool", 2, 0, 2) on planes of even height and width ->
    ("bnrelupool", name, C)."""
    shapes = layer_shapes(spec, input_shape) if pool else None
    out, i = [], 0
    while i < len(spec):
        if spec[i][0] == "bn" and i + 1 < len(spec) and spec[i + 1][0] == "relu":
            if (pool and i + 2 < len(spec) and tuple(spec[i + 2]) == ("maxpool", 2, 0, 2) and shapes[i][2] % 2 == 0
                    and shapes[i][3] % 2 == 0):
                out.append(("bnrelupool",) + tuple(spec[i][1:]))
                i += 3
                continue
            out.append(("bnrelu",) + tuple(spec[i][1:]))
            i += 2
        else:
            out.append(spec[i])
            i += 1
    return out


def layer_shapes(spec, input_shape):
    from .trainer import _out_shape
    shapes = [tuple(input_shape)]
    for layer in spec:
        shapes.append(_out_shape(layer, shapes[-1]))
    return shapes


def tensor_bytes(shapes):
    return [4 * int(math.prod(s)) for s in shapes]


def default_issue_at(swap, n_layers, prefetch):
    """tensor -> backward layer at whose start its copy-in is issued: `prefetch` layers ahead."""
    return {j: min(n_layers - 1, j + prefetch) for j in swap}


def simulate(spec, shapes, swap=(), fixed_bytes=0, prefetch=3, issue_at=None, recompute=()):
    """Replays the executor's allocation schedule.  Returns (peak_bytes, events) where events is
    a list of (phase, layer, resident_bytes, resident_tensor_indices, busy_tensor_indices); phase
    "re" is the moment tensor `layer` has just been computed again."""
    L = len(spec)
    size = tensor_bytes(shapes)
    swap = set(swap)
    redo = set(recompute)
    issue_at = issue_at if issue_at is not None else default_issue_at(swap, L, prefetch)
    resident = set([0])
    grad_bytes = 0
    events = []

    def note(phase, li):
        events.append((phase, li, fixed_bytes + sum(size[j] for j in resident) + grad_bytes, frozenset(resident),
                       frozenset((li, li + 1))))

    for li in range(L):
        resident.add(li + 1)
        note("fwd", li)
        if li in swap or li in redo:
            resident.discard(li)
    g_out = size[L]                    # the loss gradient has the logits' size
    grad_bytes = g_out
    for li in range(L - 1, -1, -1):
        # only max pooling reads its own output in the backward pass; every other layer's output is dead
        # as soon as the layer behind it has been through, before anything is allocated for this one
        if spec[li][0] not in NEEDS_OUTPUT_BACKWARD:
            resident.discard(li + 1)
        # copy-ins issued at the start of this layer's backward (its own input at the latest)
        for j in swap:
            if 1 <= j <= li + 1 and (issue_at[j] >= li or j >= li):
                resident.add(j)
        # this layer's input, if it was dropped, is computed again (and what it is computed from first)
        chain = []
        j = li
        while j in redo and j not in resident:
            chain.append(j)
            j -= 1
        for j in reversed(chain):
            resident.add(j)
            events.append(("re", j, fixed_bytes + sum(size[k] for k in resident) + grad_bytes, frozenset(resident),
                           frozenset((j - 1, j))))
        in_place = spec[li][0] in IN_PLACE_BACKWARD
        g_in = 0 if li == 0 else g_out if in_place else size[li]
        grad_bytes = g_out if (li == 0 or in_place) else g_out + g_in
        note("bwd", li)
        resident.discard(li + 1)
        g_out = g_in
        grad_bytes = g_out
    peak = max(e[2] for e in events)
    return peak, events


def layer_times(spec, shapes, cost):
    """-> (forward ms, backward ms) per layer under `cost`; `step_ms` takes them ready-made when
    it is called many times for one net."""
    L = len(spec)
    return ([cost.layer_ms(spec[li], shapes[li], shapes[li + 1], False) for li in range(L)],
            [cost.layer_ms(spec[li], shapes[li], shapes[li + 1], True, first=li == 0) for li in range(L)])


def step_ms(spec, shapes, swap, cost, prefetch=3, issue_at=None, recompute=(), budget_bytes=None, fixed_bytes=0,
            times=None):
    """Estimated step time under the replayed schedule: one compute stream, one copy-out and one
    copy-in stream (each link direction carries one copy at a time, in issue order).  A swapped
    tensor starts leaving when its consumer starts; its memory comes back when both the consumer
    and the copy are done, and releases are handed back in the order they were made.  As in the
    executor, nothing waits for a release until an allocation would not fit `budget_bytes` without
    it (no budget: never), except at the turn, where the backward sweep starts only after every
    copy-out has finished.  A copy-in is issued `prefetch` layers ahead (or where `issue_at` says)
    and the layer that needs the tensor waits for its arrival."""
    L = len(spec)
    size = tensor_bytes(shapes)
    fwd_ms, bwd_ms = times if times is not None else layer_times(spec, shapes, cost)
    swap, redo = set(swap), set(recompute)
    issue_at = issue_at if issue_at is not None else default_issue_at(swap, L, prefetch)
    clock = [0.0, fixed_bytes + size[0]]      # compute-stream time (ms), bytes held
    pending = collections.deque()             # (bytes, time the release is through), in order of release

    def alloc(nbytes):
        while pending:
            held, ready = pending[0]
            if ready > clock[0]:
                if budget_bytes is None or clock[1] + nbytes <= budget_bytes:
                    break
                clock[0] = ready              # the allocation waits for the oldest release
            pending.popleft()
            clock[1] -= held
        clock[1] += nbytes

    def release(nbytes, ready=0.0):
        pending.append((nbytes, max(clock[0], ready)))

    out_free = 0.0
    for li in range(L):
        alloc(size[li + 1])
        started = clock[0]
        clock[0] += fwd_ms[li]
        if li in swap:
            out_free = max(out_free, started) + cost.copy_ms(size[li])
            release(size[li], out_free)
            clock[0] += cost.host_wait_ms
        elif li in redo:
            release(size[li])
    while pending:                            # the turn: every tensor that left has really left
        held, ready = pending.popleft()
        clock[0] = max(clock[0], ready)
        clock[1] -= held
    alloc(size[L])
    g_out = size[L]
    in_free, arrival = 0.0, {}
    away, dropped = set(j for j in swap if j >= 1), set(redo)
    here = set(range(L + 1)) - away - dropped
    for li in range(L - 1, -1, -1):
        if spec[li][0] not in NEEDS_OUTPUT_BACKWARD and li + 1 in here:
            here.discard(li + 1)
            release(size[li + 1])
        for j in sorted(away, reverse=True):          # the tensor needed first is issued first
            if issue_at[j] >= li or j >= li:
                away.discard(j)
                here.add(j)
                alloc(size[j])
                in_free = max(in_free, clock[0]) + cost.copy_ms(size[j])
                arrival[j] = in_free
                clock[0] += cost.host_wait_ms
        chain = []
        j = li
        while j in dropped:
            chain.append(j)
            j -= 1
        for j in reversed(chain):                     # every dropped tensor is computed again once
            dropped.discard(j)
            here.add(j)
            alloc(size[j])
            clock[0] += fwd_ms[j - 1]
        in_place = spec[li][0] in IN_PLACE_BACKWARD
        g_in = 0 if li == 0 else g_out if in_place else size[li]
        if li and not in_place:
            alloc(g_in)
        clock[0] = max(clock[0], arrival.get(li, 0.0)) + bwd_ms[li]
        if li + 1 in here:
            here.discard(li + 1)
            release(size[li + 1])
        if not in_place or li == 0:
            release(g_out)
        g_out = g_in
    return clock[0]


def plan_memory(spec, input_shape, budget_bytes=None, fixed_bytes=0, cost=None, piece_bytes=128 << 20, prefetch=3,
                allow_recompute=False):
    """-> MemoryPlan for `spec` (already fused, if fusion is wanted).  Raises ValueError when
    even removing every idle tensor does not fit the budget.  With `allow_recompute` an idle
    tensor that a BatchNorm / Relu layer produced may also be dropped and computed again in the
    backward sweep instead of travelling to the host and back; the planner takes whichever of the
    two adds less estimated step time per byte freed."""
    cost = cost or CostModel()
    shapes = layer_shapes(spec, input_shape)
    batch = shapes[0][0]
    size = tensor_bytes(shapes)
    L = len(spec)
    swap, redo = set(), set()

    def replay(sw, rd, issue=None):
        return simulate(spec, shapes, sw, fixed_bytes, prefetch, issue, rd)

    times = layer_times(spec, shapes, cost)

    def est(sw, rd, issue=None):
        return step_ms(spec, shapes, sw, cost, prefetch, issue, rd, budget_bytes, fixed_bytes, times)

    def may_redo(j):
        # produced by a cheap layer, and what it is computed from stays on the device
        if not allow_recompute or j < 1 or j >= L or spec[j - 1][0] not in CHEAP_TO_REDO:
            return False
        k = j - 1
        while k in redo:
            k -= 1
        return k not in swap

    def early_issue(swap, redo, now_ms, peak):
        # copy-ins may start earlier than `prefetch` layers ahead where the budget has room for the
        # tensor over the whole stretch; the order of issue stays the order of need
        issue_at = default_issue_at(swap, L, prefetch)
        if budget_bytes is not None and swap:
            bound = L - 1
            for j in sorted(swap, reverse=True):
                best_at = issue_at[j]
                for at in range(issue_at[j] + 1, bound + 1):
                    trial = dict(issue_at)
                    trial[j] = at
                    if replay(swap, redo, trial)[0] > budget_bytes:
                        break
                    best_at = at
                issue_at[j] = best_at
                bound = best_at
            now_ms = est(swap, redo, issue_at)
            peak = replay(swap, redo, issue_at)[0]
        return now_ms, peak, issue_at

    free_ms = est(set(), set())

    def choose(power):
        """One greedy pass scoring a candidate by added time / size**power -> (ms, peak, issue_at, swap, redo)."""
        swap.clear()
        redo.clear()
        now_ms = free_ms
        while True:
            peak, events = replay(swap, redo)
            if budget_bytes is None or peak <= budget_bytes:
                break
            # moments at the peak; candidates = resident, idle, still kept, neither batch nor logits
            candidates, coming_back = set(), set()
            for phase, li, total, resident, busy in events:
                if total < peak:
                    continue
                for j in resident - busy - swap - redo:
                    if j == 0 or j >= L:
                        continue
                    candidates.add(j)
                    if phase != "fwd" and li - prefetch <= j < li:
                        coming_back.add(j)  # swapped, it would be on its way back in at that moment: only dropping helps
            best = None
            for j in candidates:
                options = []
                if j + 1 not in redo and j not in coming_back:   # a tensor something is recomputed from stays on the device
                    options.append(("swap", est(swap | {j}, redo)))
                if may_redo(j):
                    options.append(("redo", est(swap, redo | {j})))
                for how, ms in options:
                    score = (ms - now_ms + 1e-3) / float(size[j]) ** power
                    if best is None or score < best[0]:
                        best = (score, j, how)
            if best is None:
                raise ValueError("budget of %.2f GiB cannot be met: %.2f GiB are needed with every idle tensor removed"
                                 % (budget_bytes / GiB, peak / GiB))
            (redo if best[2] == "redo" else swap).add(best[1])
            now_ms = est(swap, redo)
        # the last pick may have freed more than was missing: put back what the budget can hold,
        # dearest first
        for _ in range(len(swap) + len(redo)):
            gains = []
            for j in swap:
                rest = swap - {j}
                if replay(rest, redo)[0] <= budget_bytes:
                    gains.append((now_ms - est(rest, redo), 0, j))
            for j in redo:
                rest = redo - {j}
                if replay(swap, rest)[0] <= budget_bytes:
                    gains.append((now_ms - est(swap, rest), 1, j))
            if not gains or max(gains)[0] <= 0:
                break
            _, which, j = max(gains)
            (redo if which else swap).discard(j)
            now_ms = est(swap, redo)
            peak = replay(swap, redo)[0]
        return early_issue(set(swap), set(redo), now_ms, peak) + (set(swap), set(redo))

    # time per byte freed is the natural score; weighting size less or more sometimes finds a cheaper set
    # (fewer, larger tensors that hide behind long layers), so the estimate decides between a few passes
    powers = (1.0,) if budget_bytes is None else (1.0, 0.5, 1.5)
    passes, refusal = [], None
    for pw in powers:
        try:
            passes.append(choose(pw))
        except ValueError as e:
            refusal = refusal or e
    if not passes:
        raise refusal
    now_ms, peak, issue_at, swap, redo = min(passes, key=lambda r: (r[0], len(r[3]) + len(r[4])))
    split = {}
    for li, layer in enumerate(spec):
        if layer[0] == "conv" and li >= 1 and li in swap:
            k = int(min(batch, max(1, -(-size[li] // piece_bytes))))
            if k > 1:
                split[li] = k
    return MemoryPlan(swap, split, peak, now_ms, free_ms, fixed_bytes, budget_bytes, prefetch, issue_at, redo)
