"""Named wall-clock timers and the autograd marker op the conv layers call
(cxgnncomp/timer.py:7-164).  Timers are created skipped (no-ops) exactly as
upstream; ``get_timers()`` needs ``set_timers()`` first."""
import time

import torch

_GLOBAL_TIMERS = None


class _Timer:

    def __init__(self, name):
        self.name_ = name
        self.elapsed_ = 0.0
        self.num_call = 0
        self.started_ = False
        self.start_time = time.time()
        self.input_shape = None
        self.output_shape = None
        self.skip = True

    def start(self):
        if self.skip:
            return
        assert not self.started_, "timer" + self.name_ + "has already been started"
        torch.cuda.synchronize()
        self.start_time = time.time()
        self.started_ = True

    def stop(self):
        if self.skip:
            return
        assert self.started_, "timer" + self.name_ + " is not started"
        torch.cuda.synchronize()
        self.elapsed_ += time.time() - self.start_time
        self.num_call += 1
        self.started_ = False

    def reset(self):
        if self.skip:
            return
        self.elapsed_ = 0.0
        self.started_ = False
        self.num_call = 0

    def elapsed(self, reset=True):
        if self.skip:
            return
        assert not self.started_, "timer" + self.name_ + "is still started"
        out = (self.elapsed_, self.num_call)
        if reset:
            self.reset()
        return out


class Timers:

    def __init__(self):
        self.timers = {}

    def __call__(self, name):
        if name not in self.timers:
            self.timers[name] = _Timer(name)
        return self.timers[name]

    def log(self, log_fn, names, normalizer=1.0, reset=True):
        assert normalizer > 0.0
        parts = ["time (ms)"]
        for name in names:
            ms = 0
            if name in self.timers:
                got = self.timers[name].elapsed(reset=reset)
                ms = got[0] * 1000.0 / normalizer if got else 0
            parts.append("{}: {:.2f}".format(name, ms))
        log_fn(" | ".join(parts))

    def log_all(self, log_fn, normalizer=1.0, reset=True):
        assert normalizer > 0.0
        parts = ["time (ms)"]
        for name in sorted(self.timers):
            t = self.timers[name]
            got = t.elapsed(reset=reset)
            ms = got[0] * 1000.0 / got[1] if got and got[1] else 0.0
            text = "{}: {:.2f}".format(name, ms)
            if t.input_shape is not None:
                text += "| {}: in:{} out:{}".format(name, t.input_shape, t.output_shape)
            parts.append(text)
        log_fn(" | ".join(parts))


def set_timers():
    global _GLOBAL_TIMERS
    _GLOBAL_TIMERS = Timers()


def get_timers():
    assert _GLOBAL_TIMERS is not None
    return _GLOBAL_TIMERS


class TimerOP(torch.autograd.Function):
    """Identity in value; starts/stops ``<name>_fwd`` in forward and ``<name>_bwd``
    (in the opposite order) in backward."""

    @staticmethod
    def forward(ctx, input, timer_name, is_front):
        timers = get_timers()
        if is_front:
            timers(timer_name + "_fwd").start()
        else:
            timers(timer_name + "_fwd").stop()
        ctx.timer_name = timer_name
        ctx.is_front = is_front
        return input

    @staticmethod
    def backward(ctx, grad_in):
        timers = get_timers()
        name = ctx.timer_name + "_bwd"
        if ctx.is_front:
            timers(name).stop()
        else:
            timers(name).start()
        return grad_in, None, None


class TimerModule(torch.nn.Module):

    def __init__(self, model, timer_name, report_shape=False):
        super().__init__()
        self.model = model
        self.timer_name = timer_name
        self.report_shape = report_shape

    def forward(self, input):
        input = TimerOP.apply(input, self.timer_name, True)
        output = self.model(input)
        output = TimerOP.apply(output, self.timer_name, False)
        if self.report_shape:
            t = get_timers()(self.timer_name + "_shape")
            t.input_shape = input.shape
            t.output_shape = output.shape
        return output
