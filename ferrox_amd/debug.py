"""Probes and switches for tests and measurement.  Nothing on the product path sets them; a
part looks at `routing_trace` only where it has expert choices to report.

* `trace_routing()`: while it is active every sparse feed-forward copies the experts it chose
  into a device buffer that the trace owns (one per call of a step, in the order of the
  calls).  The copy is a launch like any other, so it is also part of a recorded (HIP graph)
  decode step and is repeated by every replay; `RoutingTrace.read()` gives the last step's
  choices.  Recorded steps are kept apart by `graph_token()`: a step recorded without a trace
  is never replayed while one is active, nor the other way round.
* `region(name)`: the parts bracket their stages with it ("qkv", "attention", "experts gate/up", ...).  It
  does nothing unless `region_sink` is set; a sink is called with the name when a stage begins (bench.py sets
  one that launches a marker kernel, so that a profiler's kernel trace can be cut into stages).
* `kernel_switch(library, key, value)`: forces a kernel variant that the sizes would otherwise
  choose (the libraries' `fx_debug_set`), for tests that run every variant on the same input
  and for A/B timing; the default is restored on exit.
"""
from __future__ import annotations

import contextlib
import ctypes

import torch

KERNEL_SWITCH_DEFAULTS = {("gemm", "skinny_sets"): 0, ("gemm", "skinny_row_tiles"): 0, ("gemm", "skinny_waves"): 0, ("gemm", "few_rows"): 3, ("gemm", "head_rows"): 16, ("gemm", "tile64_rows"): 20,
                          ("gemm", "wide"): 1, ("gemm", "wide_grouped"): 0, ("gemm", "stream_w"): -1, ("gemm", "plain_rows"): 0, ("attention", "direct_stages"): 2, ("attention", "direct_groups"): 0}


class RoutingTrace:
    _serial = 0

    def __init__(self):
        RoutingTrace._serial += 1
        self.token = RoutingTrace._serial
        self._pool: list = []             # per call of a step: int32 [rows, top_k]; never freed while the trace lives
        self._retired: list = []          # (a recorded step may hold the address)
        self._calls: list = []            # the last step's (buffer, tokens), in the order of the calls

    def begin_step(self) -> None:
        self._calls = []

    def put(self, ids: torch.Tensor) -> None:
        """Called by a sparse feed-forward with its int32 [T, k] choices."""
        i = len(self._calls)
        T, k = ids.shape
        if i == len(self._pool):
            self._pool.append(None)
        buf = self._pool[i]
        if buf is None or buf.shape[0] < T or buf.shape[1] != k:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("routing trace: a buffer would have to grow while a step is being recorded")
            if buf is not None:
                self._retired.append(buf)
            buf = self._pool[i] = torch.zeros((max(T, 64), k), dtype=torch.int32, device=ids.device)
        buf[:T].copy_(ids)
        self._calls.append((buf, T))

    def calls(self) -> list:
        """What a recorded step keeps: its replays write the same buffers again."""
        return list(self._calls)

    def replayed(self, calls: list) -> None:
        self._calls = list(calls)

    def read(self) -> list:
        """[call][token][slot] of the last step (host lists); waits for the device."""
        return [buf[:T].cpu().tolist() for buf, T in self._calls]


routing_trace: RoutingTrace | None = None
region_sink = None            # callable(name) or None


def region(name: str) -> None:
    """A stage of a part begins (everything launched from here to the next call belongs to it)."""
    if region_sink is not None:
        region_sink(name)


def graph_token() -> int:
    """What a recorded step depends on beside its sizes: 0, or the active trace."""
    return routing_trace.token if routing_trace is not None else 0


@contextlib.contextmanager
def trace_routing():
    global routing_trace
    before, routing_trace = routing_trace, RoutingTrace()
    try:
        yield routing_trace
    finally:
        routing_trace = before


@contextlib.contextmanager
def kernel_switch(library: str, key: str, value: int):
    from .csrc.build import load_library
    if (library, key) not in KERNEL_SWITCH_DEFAULTS:
        raise KeyError(f"no kernel switch {library}.{key} (known: {sorted(KERNEL_SWITCH_DEFAULTS)})")
    lib = load_library(library)
    lib.fx_debug_set.argtypes = [ctypes.c_char_p, ctypes.c_int]
    lib.fx_debug_set.restype = ctypes.c_int
    if lib.fx_debug_set(key.encode(), int(value)):
        raise RuntimeError(lib.fx_last_error().decode())
    try:
        yield
    finally:
        lib.fx_debug_set(key.encode(), KERNEL_SWITCH_DEFAULTS[(library, key)])
