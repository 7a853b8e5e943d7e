"""``compare`` and ``prof`` helpers (cxgnncomp/codegen/util.py:5-32).  ``prof`` times
with HIP events on the current stream instead of triton.testing.do_bench and
returns the same kind of 3-tuple in milliseconds: (median, 20th percentile,
80th percentile); callers such as the tuner read element 1."""
import torch

global_res = []


def compare(output1, output2):
    assert output1.shape == output2.shape, f"{output1.shape} != {output2.shape}"
    close = torch.isclose(output1, output2, atol=1e-2, rtol=1e-2)
    if bool(close.all()):
        print("CORRECT: match")
    else:
        print("ERROR: differ\n==========")
        print(f"ERROR: differ ratio: {torch.sum(~close) / torch.numel(close)}\n==========")


def _bench(func, warmup=3, rep=10):
    for _ in range(warmup):
        func()
    torch.cuda.synchronize()
    times = []
    for _ in range(rep):
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        func()
        end.record()
        end.synchronize()
        times.append(start.elapsed_time(end))
    t = torch.tensor(times, dtype=torch.float64)
    q = torch.quantile(t, torch.tensor([0.5, 0.2, 0.8], dtype=torch.float64))
    return (float(q[0]), float(q[1]), float(q[2]))


def prof(task_name, method, func, display=True, log=True):
    output = _bench(func)
    if display:
        print(f"{task_name} {method}:", output)
    if log:
        global_res.append(output)
    return output
