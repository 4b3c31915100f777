"""Single-GPU stand-ins for the ring transport of the reference
(lv_xattn/async_communication.py there).

On one MI355X there is no neighbour to exchange query blocks with: the P
"ranks" of the sequence-parallel group become P rounds of an on-device loop.
The names callers import survive (lv_xattn/__init__.py:1-2 of the reference,
plus the size / rank / destroy helpers); they keep their call signatures and do the little that is left to
do: pick the device, remember P, drop cached workspaces.
"""
from __future__ import annotations

import os
from typing import Dict, Optional, Tuple

import torch

_ROUNDS = 1
_INITIALISED = False
_WORKSPACES: Dict[Tuple, torch.Tensor] = {}


class _RoundGroup:
    """What `get_sequence_parallel_group()` hands out: the emulated group of P
    members of which this GPU plays all, one per round."""

    def __init__(self, rounds: int):
        self._rounds = rounds

    def size(self) -> int:
        return self._rounds

    def rank(self) -> int:
        return 0


def initialize_distributed(rounds: Optional[int] = None) -> None:
    """Reference: reads RANK/WORLD_SIZE/LOCAL_RANK and starts NCCL
    (async_communication.py:38-59).  Here: selects the GPU and fixes the number
    of query-block rounds (argument, else LVX_ROUNDS, else WORLD_SIZE, else 1).
    No process group is created and no environment variable is required."""
    global _ROUNDS, _INITIALISED
    if rounds is None:
        rounds = int(os.environ.get("LVX_ROUNDS", os.environ.get("WORLD_SIZE", "1")))
    if rounds < 1:
        raise ValueError("rounds must be >= 1")
    _ROUNDS = rounds
    if torch.cuda.is_available():
        torch.cuda.set_device(int(os.environ.get("LOCAL_RANK", "0")) % torch.cuda.device_count())
    _INITIALISED = True


def get_sequence_parallel_group() -> _RoundGroup:
    return _RoundGroup(_ROUNDS)


def get_sequence_parallel_size() -> int:
    return _ROUNDS


def get_sequence_parallel_rank() -> int:
    return 0


def destroy_sequence_parallel() -> None:
    """Reference: drops the process group (async_communication.py:205-208).
    Here: back to one round, cached workspaces freed."""
    global _ROUNDS, _INITIALISED
    _ROUNDS, _INITIALISED = 1, False
    _WORKSPACES.clear()


def reset_global_memory_buffer(*_ignored) -> None:
    """Reference: forgets the global double buffers so the next call may use
    other shapes (async_communication.py:144-156).  Here: frees the cached
    workspaces (fp32 accumulators, split partials)."""
    _WORKSPACES.clear()


def workspace(tag: str, shape, dtype, device) -> torch.Tensor:
    """A cached scratch tensor; contents are undefined on return."""
    key = (tag, tuple(shape), dtype, str(device))
    t = _WORKSPACES.get(key)
    if t is None:
        t = torch.empty(*shape, dtype=dtype, device=device)
        _WORKSPACES[key] = t
    return t
