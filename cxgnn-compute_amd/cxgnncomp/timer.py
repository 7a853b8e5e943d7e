"""Named stage timers behind the reference's names (cxgnncomp/timer.py): ``set_timers()`` installs
a process-wide ``Timers`` registry, ``get_timers()`` returns it (and asserts that it was installed),
``TimerOP`` is an identity autograd function that opens / closes the stage ``<name>_fwd`` in the
forward pass and ``<name>_bwd`` in the backward pass, ``TimerModule`` wraps a module in such a pair.

Every stopwatch starts out with ``skip = True`` and then costs nothing: no device synchronisation,
no clock read.  Clearing ``skip`` on a stopwatch makes it measure wall-clock seconds between
``start()`` and ``stop()``, each taken after the device has drained.  The report lines keep the
reference's layout, ``time (ms) | <name>: <milliseconds per call>``.
"""
import time

import torch

_GLOBAL_TIMERS = None


def _drain_device():
    if torch.cuda.is_available() and torch.cuda.is_initialized():
        torch.cuda.synchronize()


class _Stopwatch:
    """Accumulated wall time and number of completed start/stop pairs of one named stage."""

    def __init__(self, name):
        self.name = name
        self.skip = True
        self.total_s = 0.0
        self.num_call = 0
        self.opened_at = None          # perf_counter() of the pending start(), None when closed
        self.input_shape = None
        self.output_shape = None

    @property
    def running(self):
        return self.opened_at is not None

    def start(self):
        if self.skip:
            return
        assert not self.running, "timer %s was started twice" % self.name
        _drain_device()
        self.opened_at = time.perf_counter()

    def stop(self):
        if self.skip:
            return
        assert self.running, "timer %s was stopped without a start" % self.name
        _drain_device()
        self.total_s += time.perf_counter() - self.opened_at
        self.num_call += 1
        self.opened_at = None

    def reset(self):
        if self.skip:
            return
        self.total_s, self.num_call, self.opened_at = 0.0, 0, None

    def elapsed(self, reset=True):
        """(seconds, calls) accumulated so far, or None while the stopwatch is skipping."""
        if self.skip:
            return None
        assert not self.running, "timer %s is still running" % self.name
        result = (self.total_s, self.num_call)
        if reset:
            self.reset()
        return result


class Timers:
    """Registry of stopwatches; calling it with a name returns (and on first use creates) one."""

    def __init__(self):
        self.timers = {}

    def __call__(self, name):
        watch = self.timers.get(name)
        if watch is None:
            watch = self.timers[name] = _Stopwatch(name)
        return watch

    @staticmethod
    def _ms_per(watch, divisor, reset):
        got = watch.elapsed(reset=reset) if watch is not None else None
        if got is None:
            return 0.0
        seconds, calls = got
        d = calls if divisor is None else divisor
        return seconds * 1000.0 / d if d else 0.0

    def log(self, log_fn, names, normalizer=1.0, reset=True):
        """One line with the given stages, milliseconds divided by ``normalizer``."""
        assert normalizer > 0.0
        parts = ["time (ms)"]
        for name in names:
            parts.append("%s: %.2f" % (name, self._ms_per(self.timers.get(name), normalizer, reset)))
        log_fn(" | ".join(parts))

    def log_all(self, log_fn, normalizer=1.0, reset=True):
        """One line with every stage in name order, milliseconds per completed call; stages that
        recorded shapes (TimerModule(report_shape=True)) append them."""
        assert normalizer > 0.0
        parts = ["time (ms)"]
        for name in sorted(self.timers):
            watch = self.timers[name]
            item = "%s: %.2f" % (name, self._ms_per(watch, None, reset))
            if watch.input_shape is not None:
                item += "| %s: in:%s out:%s" % (name, watch.input_shape, watch.output_shape)
            parts.append(item)
        log_fn(" | ".join(parts))


def set_timers():
    global _GLOBAL_TIMERS
    _GLOBAL_TIMERS = Timers()


def get_timers():
    assert _GLOBAL_TIMERS is not None, "call set_timers() first"
    return _GLOBAL_TIMERS


class TimerOP(torch.autograd.Function):
    """``TimerOP.apply(tensor, name, is_front)`` returns ``tensor``.  The front marker opens
    ``<name>_fwd`` and the back marker closes it; in the backward pass, which meets the markers in
    the opposite order, the back marker opens ``<name>_bwd`` and the front marker closes it."""

    @staticmethod
    def forward(ctx, input, timer_name, is_front):
        watch = get_timers()(timer_name + "_fwd")
        if is_front:
            watch.start()
        else:
            watch.stop()
        ctx.stage = (timer_name, is_front)
        return input

    @staticmethod
    def backward(ctx, grad):
        name, is_front = ctx.stage
        watch = get_timers()(name + "_bwd")
        if is_front:
            watch.stop()
        else:
            watch.start()
        return grad, None, None


class TimerModule(torch.nn.Module):
    """``model`` bracketed by a TimerOP pair named ``timer_name``; with ``report_shape`` the input
    and output shapes are kept on the stage ``<timer_name>_shape``."""

    def __init__(self, model, timer_name, report_shape=False):
        super().__init__()
        self.model = model
        self.timer_name = timer_name
        self.report_shape = report_shape

    def forward(self, input):
        input = TimerOP.apply(input, self.timer_name, True)
        output = TimerOP.apply(self.model(input), self.timer_name, False)
        if self.report_shape:
            watch = get_timers()(self.timer_name + "_shape")
            watch.input_shape, watch.output_shape = input.shape, output.shape
        return output
