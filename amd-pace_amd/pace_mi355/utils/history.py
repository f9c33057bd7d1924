"""A seeded serving history for a block allocator: what the free list of a paged KV pool looks like after
sequences have been admitted and retired for a while.  Used to set up fragmented pools (benchmarks, tests)."""
from __future__ import annotations

import math

import numpy as np


def alloc_free_history(alloc, seed, lo_blocks, hi_blocks, occupancy=0.75, turnover=4.0):
    """Leave the free list in the order a serving history leaves it in: sequences of lo..hi blocks (log-uniform)
    are admitted while the pool is below `occupancy` and retired at random, until `turnover` times the pool has
    been handed out; then the survivors retire in random order.  Seeded."""
    rng = np.random.default_rng(seed)
    live, handed = [], 0
    while handed < turnover * alloc.num_blocks:
        used = alloc.num_blocks - alloc.num_free
        n = int(round(math.exp(rng.uniform(math.log(lo_blocks), math.log(hi_blocks)))))
        if used + n <= occupancy * alloc.num_blocks and (not live or rng.random() < 0.7):
            live.append(alloc.allocate(n))
            handed += n
        elif live:
            alloc.free(live.pop(int(rng.integers(len(live)))))
    for i in rng.permutation(len(live))[::-1]:
        alloc.free(live[i])
