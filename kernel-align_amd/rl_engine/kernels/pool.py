"""Pre-allocated device workspace pool.

The reference advertises a pre-allocated chunk pool of constant size (about
0.5 GB over the resident tensors, README.md:25,34) although its compute_logp
(rl_engine/kernels/sampling.py:96-112) only pre-allocates the [G, L] output.
Here the one-pass logprob kernel needs no temporary of logits size at all, so
the pool holds only the small scratch buffers of the other kernels (sampling
histograms, fused lm_head partials).  It is one arena, allocated once per device
and handed out by a bump pointer; on a 288 GB MI355X the default 64 MiB is
0.02 % of HBM and the hard limit stays at 0.5 GB.

Sharing rule.  Operators take their scratch through ``lease``: the pool's lock is
held from the reservation to the end of the launch, so two host threads never
hold the same bytes, and every lease leaves an event on the stream it was used
on.  A later lease on another stream first makes that stream wait for the event,
so kernels of two streams never work in the arena at the same time (they run one
after the other; results are those of sequential calls).

HIP-graph capture.  A lease taken while the current stream is capturing does not
touch the arena or the events (waiting for an event recorded outside the capture,
or leaving a capture-recorded event for eager streams, is not valid, and a replay
would use the arena without any ordering against eager calls): it hands out memory
allocated under the capture, which belongs to the graph's own memory pool.  A
captured operator therefore owns its scratch; replays of the graph and eager calls
on other streams never share bytes.
"""
from __future__ import annotations

import os
import threading
from contextlib import contextmanager

import torch

DEFAULT_POOL_BYTES = 64 << 20
MAX_POOL_BYTES = 512 << 20
ENV_POOL_BYTES = "RL_ENGINE_POOL_BYTES"
ALIGN = 256


class PoolExhausted(RuntimeError):
    """A request does not fit the pre-allocated pool; the pool never grows silently."""


class WorkspacePool:
    def __init__(self, capacity_bytes: int | None = None):
        if capacity_bytes is None:
            capacity_bytes = int(os.environ.get(ENV_POOL_BYTES, DEFAULT_POOL_BYTES))
        if not 0 < capacity_bytes <= MAX_POOL_BYTES:
            raise ValueError(f"pool capacity {capacity_bytes} B outside (0, {MAX_POOL_BYTES}]")
        self.capacity = (capacity_bytes + ALIGN - 1) // ALIGN * ALIGN
        self._arenas: dict = {}  # device index -> uint8 tensor
        self._offset = 0
        self._lock = threading.RLock()
        self._last_use: dict = {}  # device index -> (raw stream handle, event recorded behind the last lease)

    def arena(self, device: torch.device) -> torch.Tensor:
        index = device.index if device.index is not None else torch.cuda.current_device()
        buf = self._arenas.get(index)
        if buf is None:
            buf = torch.empty(self.capacity, dtype=torch.uint8, device=torch.device("cuda", index))
            self._arenas[index] = buf
        return buf

    def reset(self) -> None:
        """Forget all reservations (the arena itself stays allocated)."""
        self._offset = 0

    def reserve(self, nbytes: int, device: torch.device) -> torch.Tensor:
        """Return a uint8 view of `nbytes` bytes, 256-byte aligned, valid until reset()."""
        if nbytes < 0:
            raise ValueError("negative workspace size")
        start = (self._offset + ALIGN - 1) // ALIGN * ALIGN
        if start + nbytes > self.capacity:
            raise PoolExhausted(
                f"workspace request of {nbytes} B does not fit the {self.capacity} B pool "
                f"({self._offset} B in use); raise {ENV_POOL_BYTES} (limit {MAX_POOL_BYTES})"
            )
        self._offset = start + nbytes
        return self.arena(device)[start:start + nbytes]

    @contextmanager
    def lease(self, nbytes: int, device: torch.device):
        """``with pool.lease(n, device) as ws:`` — a uint8 view of ``n`` bytes for kernels enqueued on the
        device's current stream inside the block.  Safe across streams and host threads (see the module
        docstring): the whole arena is taken, the previous user's stream is waited for, and the lock is
        released only after this user's event is recorded."""
        index = device.index if device.index is not None else torch.cuda.current_device()
        if torch.cuda.is_current_stream_capturing():
            if nbytes > self.capacity:
                raise PoolExhausted(f"workspace request of {nbytes} B exceeds the {self.capacity} B pool size")
            # graph-private memory: lives as long as the graph, used by its replays only
            yield torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=torch.device("cuda", index))[:nbytes]
            return
        with self._lock:
            self.reset()
            view = self.reserve(nbytes, device)
            stream = torch.cuda.current_stream(torch.device("cuda", index))
            last = self._last_use.get(index)
            if last is not None and last[0] != stream.cuda_stream:
                stream.wait_event(last[1])
            try:
                yield view
            finally:
                event = last[1] if last is not None else torch.cuda.Event()
                event.record(stream)
                self._last_use[index] = (stream.cuda_stream, event)

    def allocated_bytes(self) -> int:
        return self.capacity * len(self._arenas)
