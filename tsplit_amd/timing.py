"""HIP-event timing of operator launches on a given stream (events are recorded on the
stream the kernels run on, and read only after a final synchronisation)."""
import ctypes

from .stream import create_event_handle


def _raw(event):
    return ctypes.cast(event.handle.contents.handle, ctypes.POINTER(ctypes.c_void_p))[0]


class EventTimer(object):
    """Brackets operator calls with HIP events on the compute stream; elapsed times are read
    after the final synchronisation, so nothing blocks inside a step.

    chained=True: a call that begins right after another one ended on the same stream starts at
    that call's end event instead of recording its own, so back-to-back calls cost one event each
    (every event is a packet of its own in the queue, about 3 us between two kernels)."""

    def __init__(self, ctx, chained=False):
        self._mk = lambda: create_event_handle(ctx)
        self._hip = ctypes.CDLL("libamdhip64.so")
        self._pool, self._used, self.spans = [], 0, []
        self.enabled = False
        self.chained = chained
        self._last = None          # (end event, stream) of the previous call

    def _ev(self):
        if self._used == len(self._pool):
            self._pool.append(self._mk())
        self._used += 1
        return self._pool[self._used - 1]

    def begin(self, stream):
        if self.enabled:
            if self.chained and self._last is not None and self._last[1] is stream:
                self._a = self._last[0]
            else:
                self._a = self._ev()
                self._a.record(stream)

    def end(self, stream, tag, work, unit, moved=None):
        """`work` in `unit` ("flop" or "byte"); `moved`: for a call counted in FLOP, also its
        algorithmic bytes (operands read once, result written once)."""
        if self.enabled:
            b = self._ev()
            b.record(stream)
            self.spans.append((tag, work, unit, self._a, b, moved))
            self._last = (b, stream)

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float(0)
        rc = self._hip.hipEventElapsedTime(ctypes.byref(ms), ctypes.c_void_p(_raw(a)), ctypes.c_void_p(_raw(b)))
        if rc != 0:
            raise RuntimeError("hipEventElapsedTime failed: %d" % rc)
        return ms.value

    def reset(self):
        self._used, self.spans, self._last = 0, [], None

    def collect(self):
        """-> {tag: dict(calls, ms_total, ms_avg, work_per_call, unit, rate[, bytes])}; rate in TFLOP/s
        (unit "flop") or GB/s (unit "byte")"""
        out = {}
        for tag, work, unit, a, b, moved in self.spans:
            d = out.setdefault(tag, {"calls": 0, "ms_total": 0.0, "work": 0.0, "unit": unit})
            d["calls"] += 1
            d["ms_total"] += self.elapsed_ms(a, b)
            d["work"] += work
            if moved is not None:
                d["bytes"] = d.get("bytes", 0.0) + moved
        for d in out.values():
            d["ms_avg"] = d["ms_total"] / d["calls"]
            d["work_per_call"] = d["work"] / d["calls"]
            sec = d["ms_total"] * 1e-3
            d["rate"] = d["work"] / sec / (1e12 if d["unit"] == "flop" else 1e9) if sec > 0 else 0.0
        return out
