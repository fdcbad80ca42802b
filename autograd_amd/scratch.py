"""Per-node scratch layouts (counterpart of the reference's scratch.py).

The reference plans named scratch slots per op and phase and lets the arena
planner place them (scratch.py:94-145, runtime.py:306-310, 339-343).  On the HIP
device two ops need scratch, both in backward: the norm family (partial rows of
the dgamma / dbeta column reductions) and the embedding gradient (sort buffers
and carry rows).  Their sizes come from the native library.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np


@dataclass
class ScratchLayout:
    nbytes: int
    slots: dict = field(default_factory=dict)   # name -> (offset, shape, dtype)


class ScratchViews(dict):
    """name -> Storage view into the arena"""


def single_slot(name, nbytes):
    nbytes = int(nbytes)
    return ScratchLayout(nbytes=nbytes, slots={name: (0, (nbytes,), np.uint8)})


def equal_slots(names, shape, dtype):
    """several slots of one shape and storage dtype, each starting on a 256-byte boundary"""
    dtype = np.dtype(dtype)
    count = 1
    for d in shape:
        count *= int(d)
    step = (count * dtype.itemsize + 255) // 256 * 256
    slots = {name: (i * step, tuple(int(d) for d in shape), dtype) for i, name in enumerate(names)}
    return ScratchLayout(nbytes=step * len(names), slots=slots)
