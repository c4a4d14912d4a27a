"""Event timer with the semantics of the reference's `timer` (utils/perf_eval.py:21-34): a pair of
device events around the body, mean milliseconds over n, appended to recordList."""
from contextlib import contextmanager

import torch


@contextmanager
def timer(desc="Execution time", n=1, recordList=None, print_flag=True):
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    try:
        yield
    finally:
        end.record()
        torch.cuda.synchronize()
        exe_time = start.elapsed_time(end) / n
        if recordList is not None:
            recordList.append(exe_time)
        if print_flag:
            print(f"{desc}: {exe_time:5.4f} ms")
