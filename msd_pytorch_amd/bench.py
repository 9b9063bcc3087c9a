"""A ``%timeit``-style helper for timing small pieces of GPU or CPU code
(interface of the reference's msd_pytorch/bench.py:45-116: ``bench(name, timer)`` returns a
``TimeitResult`` with ``loops``, ``repeat``, ``best``, ``worst``, ``all_runs``, ``timings``,
``average`` and ``stdev``, printed as "mean +- std per loop").

``timer`` is a ``timeit.Timer`` or any callable; a callable that queues GPU work should end
with a synchronisation of its own, or be passed with ``sync=torch.cuda.synchronize``, which
is then called once per measured run (not per loop)."""
import math
import timeit


def format_time(seconds, precision=3):
    """'1.23 ms', '45.6 us', '2 min 5 s': three significant digits below a minute."""
    if seconds >= 60.0:
        parts, left = [], int(round(seconds))
        for suffix, length in (("d", 86400), ("h", 3600), ("min", 60), ("s", 1)):
            count, left = divmod(left, length)
            if count:
                parts.append(f"{count} {suffix}")
        return " ".join(parts)
    for unit, scale in (("s", 1.0), ("ms", 1e3), ("us", 1e6)):
        if seconds * scale >= 1.0:
            return f"{seconds * scale:.{precision}g} {unit}"
    return f"{seconds * 1e9:.{precision}g} ns"


class TimeitResult:
    def __init__(self, name, loops, repeat, best, worst, all_runs, precision=3):
        self.name, self.loops, self.repeat = name, loops, repeat
        self.best, self.worst, self.all_runs = best, worst, list(all_runs)
        self.timings = [t / loops for t in self.all_runs]
        self._precision = precision

    @property
    def average(self):
        return math.fsum(self.timings) / len(self.timings)

    @property
    def stdev(self):
        mean = self.average
        return math.sqrt(math.fsum((t - mean) ** 2 for t in self.timings) / len(self.timings))

    def __str__(self):
        runs = "run" if self.repeat == 1 else "runs"
        loops = "loop" if self.loops == 1 else "loops"
        return (f"{self.name + ':':<30}{format_time(self.average, self._precision):<8} +- "
                f"{format_time(self.stdev, self._precision):<8} per loop "
                f"(mean +- std. dev. of {self.repeat} {runs}, {self.loops} {loops} each)")

    __repr__ = __str__


def bench(name, timer, repeat=5, sync=None, min_time=0.2):
    """Time `timer`: the loop count grows by powers of ten until one run takes `min_time`
    seconds, then `repeat` runs of that many loops are measured."""
    if not isinstance(timer, timeit.Timer):
        fn = timer
        if sync is None:
            timer = timeit.Timer(fn)
        else:
            def once(fn=fn):
                fn()
            # the synchronisation brackets a whole run: timeit's setup statement runs before the clock starts
            class _Synced(timeit.Timer):
                def timeit(self, number=1000000):
                    sync()
                    start = timeit.default_timer()
                    for _ in range(number):
                        once()
                    sync()
                    return timeit.default_timer() - start
            timer = _Synced(once)
    loops = 1
    for power in range(10):
        loops = 10 ** power
        if timer.timeit(loops) >= min_time:
            break
    all_runs = timer.repeat(repeat, loops)
    return TimeitResult(name, loops, repeat, min(all_runs) / loops, max(all_runs) / loops, all_runs)
