"""A decode step of the paged cache captured into a HIP graph and replayed once per token.

The reference's generator runs one Python step per token (``pace/llm/generator.py:741-801``); at small batch
the GPU work of a layer (tens of microseconds) is shorter than the interpreter's work to enqueue it.  Nothing
in the library allocates, clears memory or synchronises, so the launches of a whole step -- every layer's
fused append + attention (fp32 pools: an append launch and an attention launch) -- can be captured once and
replayed with one call.  What changes from step to step
lives on the device: the caller's static q / k / v buffers, and a length counter that the graph itself advances
(``seq_len_bias_ptr`` of the attention arguments).  Everything the host would otherwise upload per step is
prepared before the capture: blocks for every future position, the block table, the work list.
"""
from __future__ import annotations

from typing import Callable, List, Optional

import numpy as np
import torch


class DecodeGraph:
    """``graph = DecodeGraph(caches, step_fn, max_steps)``; then per token: fill the static input buffers,
    ``out = graph.replay()``.

    ``caches``: the ``PagedKVCache`` layers the step touches (all layers of one ``KVCacheManager``).
    ``step_fn()``: runs one decode step on static tensors -- for every layer ``update_cache(k, v, 2)`` with
    1..32 new tokens followed by the attention call -- and returns what the caller wants back (static outputs).
    It is run once eagerly (its token is overwritten by the first replay) and once under capture.
    After ``max_steps`` replays, or any other operation on the caches, the graph is spent: build a new one.
    """

    def __init__(self, caches: List["PagedKVCache"], step_fn: Callable[[], object], max_steps: int,
                 stream: Optional[torch.cuda.Stream] = None):
        if not caches or any(c.pool is None for c in caches):
            raise RuntimeError("the caches must hold their prompt before a decode step can be captured")
        st = caches[0].state
        if any(c.state is not st for c in caches):
            raise RuntimeError("the layers of one decode graph share one block table")
        self.caches, self.state, self.max_steps, self.steps_done = caches, st, int(max_steps), 0
        self.closed = False
        self.new_tokens = 0  # tokens a step appends (set by the first update_cache of the step)
        for c in caches:
            c._flush()
        if st.tails_dirty:
            caches[0]._unshare()
        base = caches[0].lens.copy()
        if any((c.lens != base).any() for c in caches):
            raise RuntimeError("every layer must hold the same tokens when the step is captured")
        self.base = base
        dev = caches[0].pool.device
        self.counter = torch.zeros(1, dtype=torch.int32, device=dev)
        self.lens_dev = torch.from_numpy(base.astype(np.int32)).to(dev)
        self.plans = {}  # (layer-independent) attention plans by launch shape, made on first use, before the capture
        self._host = [(c.lens.copy(), c.seq_len) for c in caches]
        for c in caches:
            c._graph = self
        try:
            self._reserved = False
            side = stream or torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step_fn()                      # eager run: loads kernels, makes the plans, sizes the workspace
                if self.closed or not self._reserved:
                    raise RuntimeError("this step cannot be captured: it must be, for every layer, one update_cache of 1..32 "
                                       "tokens followed by the attention call, and nothing else on the caches")
                self._restore()
                self.counter.zero_()
                side.synchronize()
                self.graph = torch.cuda.CUDAGraph()
                self._capturing = True
                with torch.cuda.graph(self.graph, stream=side):
                    self.result = step_fn()
                    self.counter.add_(self.new_tokens)
                self._capturing = False
                self._restore()
            torch.cuda.current_stream().wait_stream(side)
        except Exception:
            # a refused capture leaves the caches as they were: whatever the failed step appended is forgotten
            self._capturing = False
            self.close()
            self._restore()
            raise

    _capturing = False

    def _restore(self) -> None:
        for c, (lens, seq_len) in zip(self.caches, self._host):
            c.lens, c.seq_len, c._pending, c._graph_appended = lens.copy(), seq_len, None, False

    def reserve(self, new_tokens: int) -> None:
        """Called by the first ``update_cache`` of the eager run: blocks and table for every future position."""
        if self._reserved:
            if new_tokens != self.new_tokens:
                raise RuntimeError("every layer of a captured step appends the same number of tokens")
            return
        if self._capturing:
            raise RuntimeError("the captured step differs from its eager run")
        self.new_tokens = int(new_tokens)
        self.state.ensure_capacity(self.base + self.new_tokens * self.max_steps)
        self.table = self.state.device_table()
        self._reserved = True

    def plan(self, key, make):
        """The work list of an attention launch shape, planned once (uploads are not capturable)."""
        if key not in self.plans:
            if self._capturing:
                raise RuntimeError("the captured step differs from its eager run")
            items, parts, n_items, max_parts, ws_bytes = make()
            # private copies: the state's own plan buffers are rewritten by the next plan
            self.plans[key] = (items.clone(), parts.clone(), n_items, max_parts, ws_bytes)
            self.state.workspace(ws_bytes)
        return self.plans[key]

    def replay(self):
        if self.closed:
            raise RuntimeError("this decode graph is spent (another cache operation ran, or max_steps were replayed): capture a new one")
        if self.steps_done >= self.max_steps:
            self.close()
            raise RuntimeError(f"the decode graph reserved blocks for {self.max_steps} steps; capture a new one")
        self.graph.replay()
        self.steps_done += 1
        for i, c in enumerate(self.caches):
            lens, seq_len = self._host[i]
            c.lens = lens + self.new_tokens * self.steps_done
            c.seq_len = seq_len + self.new_tokens * self.steps_done
        return self.result

    def close(self) -> None:
        """Hand the caches back to step-by-step operation (the tokens appended so far stay)."""
        self.closed = True
        for c in self.caches:
            if getattr(c, "_graph", None) is self:
                c._graph = None
