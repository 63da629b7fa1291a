"""Timing and acceptance helpers with the semantics of the reference's harness utilities
(``run_perftest`` tests/test_common.py:23-184, ``checkAllclose`` / ``verify_output`` :353-423), written for this
package: the timed loop rotates through deep copies of the arguments so that caches cannot serve the operands,
device time comes from HIP events on the current stream (optionally from one HIP-graph replay), and acceptance is
"fewer than 5 % of elements outside isclose, else a cosine-style distance below a threshold"."""

from __future__ import annotations

import copy

import torch


def _input_bytes(args, device_index):
    return sum(a.nbytes for a in args if isinstance(a, torch.Tensor) and a.is_cuda and a.device.index == device_index) + 1


def run_perftest(func, *args, num_iters=20, num_warmup=3, testGraph=False, num_rotate_args=0, needTrace=False, **kwargs):
    """Run ``func(*args, **kwargs)`` ``num_iters`` times over rotating argument copies; returns ``(last result, average
    microseconds per call)``.  ``num_rotate_args`` = 0 sizes the rotation so that the copies exceed the caches (capped at
    ``num_iters`` and by free memory), like the reference does."""
    dev = torch.cuda.current_device()
    n = int(num_rotate_args)
    if n < 1:
        in_bytes = _input_bytes(args, dev)
        props = torch.cuda.get_device_properties(dev)
        free = torch.cuda.mem_get_info(dev)[0]
        cache = min(getattr(props, "L2_cache_size", 4 << 20) * 64 * 128, free * 0.9)
        n = int((max(cache, 0) + in_bytes - 1) // in_bytes)
    n = max(1, min(n, int(num_iters)))
    rotate = [(copy.deepcopy(args), copy.deepcopy(kwargs)) for _ in range(n - 1)] + [(args, kwargs)]
    data = None
    for _ in range(int(num_warmup)):
        data = func(*args, **kwargs)
    torch.cuda.synchronize()

    def loop():
        out = None
        for i in range(int(num_iters)):
            a, k = rotate[i % n]
            out = func(*a, **k)
        return out

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    if testGraph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            data = loop()
        torch.cuda.synchronize()
        graph.replay()  # the first replay uploads the graph
        torch.cuda.synchronize()
        start.record()
        graph.replay()
        stop.record()
    else:
        start.record()
        data = loop()
        stop.record()
    stop.synchronize()
    return data, start.elapsed_time(stop) * 1e3 / int(num_iters)


def checkAllclose(a, b, rtol=1e-2, atol=1e-2, tol_err_ratio=0.05, msg="", printNum=8, printLog=True):
    """0 when every element is within ``atol + rtol*|b|``; otherwise the fraction of elements that is not."""
    close = torch.isclose(a, b, rtol=rtol, atol=atol)
    if bool(close.all()):
        return 0
    return float((~close).sum().item()) / a.numel()


def verify_output(c_out, c_ref, atol=1e-2, rtol=1e-2, msg="", logits_diff_threshold=2e-3):
    if checkAllclose(c_out, c_ref, rtol=rtol, atol=atol) < 0.05:
        return True
    x, y = c_out.double(), c_ref.double()
    den = (x * x + y * y).sum()
    diff = 0.0 if den == 0 else float(1 - 2 * (x * y).sum() / den)
    if diff != diff:
        diff = 1.0
    return diff <= logits_diff_threshold
