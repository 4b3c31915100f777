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
# Largest dS^T workspace one backward call may use; larger row windows are cut into chunks
# (see set_backward_workspace_cap)
_BWD_WS_CAP = int(float(os.environ.get("LVX_BWD_WS_CAP_GB", "12")) * (1 << 30))


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


def set_backward_workspace_cap(nbytes: int) -> None:
    """The backward keeps scale*dS for a whole row window in a workspace of
    2 bytes x B x Hq x Lkv (rounded up to 128) x rows: 1.7 GB at B1 Hq32 Lq4096 Lkv6404, 13.7 GB at
    B8.  A window whose workspace would exceed `nbytes` is run as several calls over row chunks
    (dK / dV accumulate in fp32 across them), which costs a few per cent per extra call.
    Default 12 GiB, or LVX_BWD_WS_CAP_GB."""
    global _BWD_WS_CAP
    if nbytes < (64 << 20):
        raise ValueError("the cap must leave room for at least one chunk of rows (64 MiB or more)")
    _BWD_WS_CAP = int(nbytes)


def backward_workspace_cap() -> int:
    return _BWD_WS_CAP


def workspace(tag: str, shape, dtype, device) -> torch.Tensor:
    """A cached scratch tensor; contents are undefined on return.  One buffer per (tag, device,
    stream), grown to the largest size asked for so far: changing shapes (variable-length
    batches) reuse it instead of adding a buffer per shape, and two streams never share one."""
    dev = torch.device(device)
    if dev.type == "cuda" and dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    stream = torch.cuda.current_stream(dev).cuda_stream if dev.type == "cuda" else 0
    key = (tag, str(dev), stream)
    numel = 1
    for n in shape:
        numel *= int(n)
    nbytes = numel * torch.empty((), dtype=dtype).element_size()
    buf = _WORKSPACES.get(key)
    if buf is None or buf.numel() < nbytes:
        _WORKSPACES.pop(key, None)
        buf = None                       # the old buffer is released before the larger one is asked for
        buf = torch.empty((nbytes + 255) // 256 * 256, dtype=torch.uint8, device=dev)
        _WORKSPACES[key] = buf
    return buf[:nbytes].view(dtype).view(*shape)
