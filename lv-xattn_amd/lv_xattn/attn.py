"""Host round loops of the cross-attention hot path, with the call signatures
of the reference's `_attn_forward` / `_attn_backward`
(lv_xattn/attn.py:297-298 and :437 there).

The reference moves each query block round a ring of P GPUs; every GPU
computes that block's partial result against its own stationary K/V shard and
folds it into the (O, LSE) accumulator travelling with the block.  On one
MI355X the P visits are P rounds over the query blocks of `q`, all against the
one local shard: round r computes block r's partial with `lvx_fwd`, then
`lvx_merge` folds it into that block's accumulator (what would have arrived
from the left neighbour: `acc_in`, default the identity (0, -inf)).

Everything runs on the current PyTorch stream; nothing here synchronises.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

from . import ops
from .async_communication import backward_workspace_cap, get_sequence_parallel_size, workspace
from .ops import Mask

__all__ = ["_attn_forward", "_attn_backward", "q_block_bounds", "Mask"]


def q_block_bounds(lq: int, rounds: int) -> List[Tuple[int, int]]:
    """Row window of each of the P query blocks: ceil(Lq/P) rows, the tail
    shorter (the reference needs Lq % P == 0: test.py:160)."""
    lb = -(-lq // rounds)
    return [(min(r * lb, lq), min((r + 1) * lb, lq)) for r in range(rounds)]


def _usable(t: torch.Tensor) -> torch.Tensor:
    """The kernels take any [B,H,S,D] view with unit last stride and the other
    strides multiples of 8 elements; anything else is copied once."""
    if t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:-1]) or t.data_ptr() % 16:
        return t.contiguous()
    return t


HEAD_DIM = 128          # the largest head dimension the kernels are built for
NATIVE_HEAD_DIMS = (16, 32, 64, 128)


def _pad_head_dim(t: torch.Tensor) -> torch.Tensor:
    """Head dimensions 16, 32, 64 and 128 (the reference's, lv_xattn/attn.py:306-311)
    have kernels.  Others below 128 run zero-padded to the next of them: the
    padded columns add nothing to q k^T, and the padded columns of O, dQ, dK and
    dV come out zero and are cut off again.  Exact, at the cost of the padded
    arithmetic."""
    D = t.shape[-1]
    if D in NATIVE_HEAD_DIMS:
        return t
    if D > HEAD_DIM:
        raise ValueError(f"head_dim {D} exceeds {HEAD_DIM}")
    out = t.new_zeros(*t.shape[:-1], min(d for d in NATIVE_HEAD_DIMS if d >= D))
    out[..., :D] = t
    return out


def _reject_unsupported(causal):
    if causal:
        # the reference applies the triangle to rank-local indices only
        # (lv_xattn/attn.py:229,237), which means nothing once blocks travel
        raise ValueError("causal=True is not defined for cross-attention over travelling query blocks: the "
                         "reference applies the triangle to rank-local row and key indices only "
                         "(lv_xattn/attn.py:229-237).  Its patched Mllama forward passes is_causal=True "
                         "whenever there is no attention mask and more than one query (test_llama3.py:430); "
                         "pass False there, cross-attention has no causal order")


def _dense_bias(bias_func, local_bias_args, remote_bias_args, B, Hq, Lq, Lkv, dev) -> Optional[torch.Tensor]:
    """The additive bias of the reference (lv_xattn/attn.py:386-389): there,
    bias_func(*(local_bias_args + remote_bias_args)) is evaluated once per round
    with the visiting block's remote arguments and yields [B, 1, Lb, Lkv].  Here
    q holds all P blocks, so the remote arguments describe all Lq rows and the
    one call yields [B|1, 1|Hq, Lq, Lkv]; every launch indexes it by absolute row."""
    if bias_func is None:
        if len(local_bias_args) or len(remote_bias_args):
            raise ValueError("bias arguments given without a bias_func")
        return None
    bias = bias_func(*(list(local_bias_args) + list(remote_bias_args)))
    if bias.dim() != 4 or tuple(bias.shape[2:]) != (Lq, Lkv) or bias.shape[0] not in (1, B) or bias.shape[1] not in (1, Hq):
        raise ValueError(f"bias_func must return [B|1, 1|Hq, {Lq}, {Lkv}], got {tuple(bias.shape)}")
    bias = bias.to(device=dev, dtype=torch.float32)
    pad = -Lkv % 4          # the kernels read a row in groups of 4 keys
    # rows are read with 16-byte loads: aligned base, strides multiples of 4, rows readable up to Lkv + pad
    strides_ok = all(bias.stride(i) % 4 == 0 or bias.shape[i] == 1 for i in range(3))
    if bias.stride(3) != 1 or bias.stride(2) < Lkv + pad or not strides_ok or bias.data_ptr() % 16:
        kept = getattr(bias, "lvx_padded", None)
        if kept is not None:
            return kept
        padded = torch.zeros(*bias.shape[:3], Lkv + pad, dtype=torch.float32, device=dev)
        padded[..., :Lkv] = bias
        view = padded[..., :Lkv]
        if getattr(bias, "lvx_reused", False):      # see _bias_and_hull: the copy is kept with it
            view.lvx_reused = True
            bias.lvx_padded = view
        bias = view
    return bias


def _bias_and_hull(bias: torch.Tensor, q, k):
    """(bias or None, interval mask) for a dense bias given without a mask.  The mask is the hull of
    what the bias leaves visible (ops.bias_hull), so the kernels skip what it masks anyway.  A bias
    whose maker keeps it for later calls (attribute `lvx_reused`, set by the Hugging Face hook on
    the mask it converts once per model call) is also tested once for being nothing but that
    interval mask - 0 wherever it is not -inf - and is then dropped: the interval-mask kernels give
    the same result without reading it.  The test waits for the GPU, which is why it is only made
    for a bias that comes back; hull and verdict stay with the tensor (and so does the padded copy
    _dense_bias may have to make of it), so a tensor marked `lvx_reused` must not be written to
    afterwards."""
    key = (tuple(q.shape[:3]), k.shape[2])
    kept = getattr(bias, "lvx_hull", None)
    if kept is not None and kept[0] == key:
        return (None if kept[2] else bias), kept[1]
    hull = ops.bias_hull(q, k, bias)
    if not getattr(bias, "lvx_reused", False):
        return bias, hull
    exact = ops.bias_is_interval(q, k, bias, hull)
    bias.lvx_hull = (key, hull, exact)
    return (None if exact else bias), hull


def auto_kv_splits(B: int, Hq: int, Hkv: int, rows: int, Lkv: int, target_wgs: int = 512) -> int:
    """Key splits for one forward launch over `rows` text rows.  A work-group
    covers 128 (row, head) pairs of one kv head (4 waves x 32 rows); a one-round
    launch (256 rows) has 64 of them on a 256-CU GPU, so the key range is cut
    into up to 8 parts (each at least 512 keys) until there are two work-groups
    per CU; the parts are folded by the merge kernel."""
    hg = math.gcd(Hq // Hkv, 4)
    wgs = B * (Hq // hg) * -(-rows // (32 * (4 // hg)))
    s = 1
    while s < 8 and wgs * s < target_wgs and Lkv // (2 * s) >= 512:
        s *= 2
    return s


def _attn_forward(q, k, v, causal, sm_scale, comm_mode, bias_func=None,
                  local_bias_args=[], remote_bias_args=[], no_overlap=False, *,
                  rounds: Optional[int] = None, mask: Optional[Mask] = None,
                  acc_in: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                  kv_splits: Optional[int] = None, batched: bool = False, streams: int = 1):
    """Returns (q, k, v, o, L) like the reference (attn.py:435): o [B,Hq,Lq,D]
    bf16, L [B*Hq, Lq] fp32 natural-log LSE of sm_scale * q k^T.

    q [B,Hq,Lq,D] holds all P query blocks back to back; k, v [B,Hkv,Lkv,D] are
    the local shard at Hkv heads (Hkv | Hq; expanded in-kernel).
    `comm_mode` and `no_overlap` are accepted and ignored (no transport).
    Keyword-only additions: `rounds` (P; default the size set by
    initialize_distributed), `mask`, `acc_in` = (O_in bf16 [B,Hq,Lq,D],
    L_in fp32 [B*Hq,Lq]) for every block, `kv_splits` (key ranges per round
    computed by separate work-groups; default: enough to give every CU two
    work-groups, see auto_kv_splits), `batched` (one launch over all P blocks
    instead of one per round), `streams` (the rounds of one call touch disjoint rows, so on one
    GPU they may overlap: round r is queued on stream r % streams, the current stream and
    streams - 1 others of the same priority, joined before the call returns)."""
    _reject_unsupported(causal)
    D_in = q.shape[-1]
    q_, k_, v_ = (_usable(_pad_head_dim(t)) for t in (q, k, v))
    B, Hq, Lq, D = q_.shape
    P = rounds if rounds is not None else get_sequence_parallel_size()
    dev = q_.device
    bias = _dense_bias(bias_func, local_bias_args, remote_bias_args, B, Hq, Lq, k_.shape[2], dev)
    if mask is not None:
        mask = mask.to(dev)
    elif bias is not None:
        bias, mask = _bias_and_hull(bias, q_, k_)    # skip what the bias masks out anyway

    o = torch.empty(B, Hq, Lq, D, dtype=q_.dtype, device=dev)
    L = torch.empty(B * Hq, Lq, dtype=torch.float32, device=dev)
    if acc_in is not None:
        acc_o = _usable(_pad_head_dim(acc_in[0].to(dtype=q_.dtype)))
        acc_l = acc_in[1].to(torch.float32).reshape(B * Hq, Lq).contiguous()

    windows = [(0, Lq)] if batched else [w for w in q_block_bounds(Lq, P) if w[1] > w[0]]
    max_rows = max(r1 - r0 for r0, r1 in windows)
    if kv_splits is None:
        kv_splits = auto_kv_splits(B, Hq, k_.shape[1], max_rows, k_.shape[2])
    ws = None
    if kv_splits > 1:
        nbytes = ops.fwd_workspace_bytes(q_, k_, max_rows, kv_splits)
        ws = workspace("fwd_split", (nbytes,), torch.uint8, dev)

    # the partial goes straight into (o, L), merged on its way with the incoming accumulator
    # if there is one (with key splits by the launch that folds the splits; neither a copy of
    # acc_in nor a buffer for the partial is needed)
    acc = (acc_o, acc_l) if acc_in is not None else None

    def one_round(r0, r1, ws):
        ops.fwd(q_, k_, v_, o, L, sm_scale, r0, r1 - r0, mask, kv_splits, ws, bias, acc=acc)

    if streams > 1 and len(windows) > 1:
        with _RoundStreams(dev, min(streams, len(windows))) as rs:
            for i, (r0, r1) in enumerate(windows):
                with rs.stream(i):
                    ws_i = workspace("fwd_split", (nbytes,), torch.uint8, dev) if kv_splits > 1 else None
                    one_round(r0, r1, ws_i)
    else:
        for r0, r1 in windows:
            one_round(r0, r1, ws)
    if D_in != D:
        o = o[..., :D_in].contiguous()
    return q, k, v, o, L


class _RoundStreams:
    """The current stream plus n - 1 side streams of the same (default) priority for the rounds
    of one call.  The side streams start behind everything queued on the current stream so far;
    on exit the current stream waits for all of them, so nothing that follows the call can see
    a half-finished round and every tensor the rounds touched may be released as usual."""
    _side = {}

    def __init__(self, device, n):
        self.dev, self.n = torch.device(device), n

    def __enter__(self):
        self.main = torch.cuda.current_stream(self.dev)
        side = _RoundStreams._side.setdefault(str(self.dev), [])
        while len(side) < self.n - 1:
            side.append(torch.cuda.Stream(self.dev))
        self.streams = [self.main] + side[:self.n - 1]
        start = self.main.record_event()
        for s in self.streams[1:]:
            s.wait_event(start)
        return self

    def stream(self, i):
        return torch.cuda.stream(self.streams[i % self.n])

    def __exit__(self, *exc):
        for s in self.streams[1:]:
            self.main.wait_event(s.record_event())
        return False


def _cap_windows(windows, nbytes_of_rows, cap):
    """Cuts every row window whose backward workspace would exceed `cap` bytes into chunks of
    whole 256-row groups that fit (the workspace grows linearly with the rows of a call)."""
    out = []
    for r0, r1 in windows:
        rows = r1 - r0
        if rows <= 256 or nbytes_of_rows(rows) <= cap:
            out.append((r0, r1))
            continue
        chunk = rows
        while chunk > 256 and nbytes_of_rows(chunk) > cap:
            chunk = max(256, (chunk // 2 + 255) // 256 * 256)
        out.extend((a, min(a + chunk, r1)) for a in range(r0, r1, chunk))
    return out


def _attn_backward(do, q, k, v, o, L, causal, sm_scale, comm_mode, backward_engine,
                   bias_func=None, local_bias_args=[], remote_bias_args=[], no_overlap=False, *,
                   rounds: Optional[int] = None, mask: Optional[Mask] = None, batched: bool = False,
                   streams: int = 1):
    """Returns (dq, dk, dv) like the reference (attn.py:545): dq [B,Hq,Lq,D];
    dk, dv [B,Hkv,Lkv,D]-shaped views of [B,Lkv,Hkv,D] memory, at the Hkv heads
    k and v came in with.  `o` and `L` are the finally merged forward results;
    every round uses them, so per-round contributions simply add
    (attn.py:465-468, 509-527).  dK, dV are summed in fp32 across the q heads of
    a group and across rounds and rounded to bf16 once; a round's dQ rows are
    complete after that round (fp32 sum over all local tokens, rounded once).
    `backward_engine`, `comm_mode`, `no_overlap` are accepted and ignored.  `streams` as in
    `_attn_forward`; every stream sums its rounds' dK, dV in an fp32 accumulator of its own and
    the accumulators are added before the one rounding."""
    _reject_unsupported(causal)
    D_in = q.shape[-1]
    q_, k_, v_, o_, do_ = (_usable(_pad_head_dim(t)) for t in (q, k, v, o, do))
    B, Hq, Lq, D = q_.shape
    Hkv, Lkv = k_.shape[1], k_.shape[2]
    P = rounds if rounds is not None else get_sequence_parallel_size()
    dev = q_.device
    bias = _dense_bias(bias_func, local_bias_args, remote_bias_args, B, Hq, Lq, Lkv, dev)
    if mask is not None:
        mask = mask.to(dev)
    elif bias is not None:
        bias, mask = _bias_and_hull(bias, q_, k_)    # as in the forward: the same hull, hence the same pairs
    L_ = L.to(torch.float32).reshape(B * Hq, Lq).contiguous()

    delta = workspace("bwd_delta", (B * Hq, Lq), torch.float32, dev)
    dq = torch.empty(B, Hq, Lq, D, dtype=q_.dtype, device=dev)
    dk = torch.empty(B, Lkv, Hkv, D, dtype=q_.dtype, device=dev).transpose(1, 2)
    dv = torch.empty(B, Lkv, Hkv, D, dtype=q_.dtype, device=dev).transpose(1, 2)

    windows = [(0, Lq)] if batched else [w for w in q_block_bounds(Lq, P) if w[1] > w[0]]
    windows = _cap_windows(windows, lambda rows: ops.bwd_workspace_bytes(q_, k_, rows, mask), backward_workspace_cap())
    ws = workspace("bwd_ds", (ops.bwd_workspace_bytes(q_, k_, max(r1 - r0 for r0, r1 in windows), mask),),
                   torch.uint8, dev)
    if len(windows) == 1:
        r0, r1 = windows[0]
        ops.bwd_preprocess(o_, do_, delta, r0, r1 - r0)
        ops.bwd(q_, k_, v_, do_, L_, delta, dq, dk, dv, sm_scale, r0, r1 - r0, mask, accumulate_dkv=False,
                workspace=ws, bias=bias)
    else:
        def accumulators():
            a = workspace("bwd_dkv_acc", (2, B, Lkv, Hkv, D), torch.float32, dev)
            a.zero_()
            return a

        # delta depends on O and dO alone, and all P blocks of both are here: one launch for
        # all rows ahead of the rounds (a visit of a real ring would bring its own block's)
        ops.bwd_preprocess(o_, do_, delta, 0, Lq)

        def one_round(r0, r1, acc, ws_r):
            ops.bwd(q_, k_, v_, do_, L_, delta, dq, acc[0].transpose(1, 2), acc[1].transpose(1, 2), sm_scale,
                    r0, r1 - r0, mask, accumulate_dkv=True, workspace=ws_r, bias=bias)

        acc = accumulators()
        n_streams = min(streams, len(windows))
        if n_streams > 1:
            ws_bytes = ws.numel()
            with _RoundStreams(dev, n_streams) as rs:
                accs = [acc]
                for j in range(1, n_streams):
                    with rs.stream(j):
                        accs.append(accumulators())      # cached per stream, like the dS^T workspace
                for i, (r0, r1) in enumerate(windows):
                    with rs.stream(i):
                        ws_i = ws if i % n_streams == 0 else workspace("bwd_ds", (ws_bytes,), torch.uint8, dev)
                        one_round(r0, r1, accs[i % n_streams], ws_i)
            for other in accs[1:]:
                acc += other
        else:
            for r0, r1 in windows:
                one_round(r0, r1, acc, ws)
        # [B,Hkv,Lkv,D] views of [B,Lkv,Hkv,D] memory: cast in memory order
        ops.cast_f32(acc[0], dk.transpose(1, 2))
        ops.cast_f32(acc[1], dv.transpose(1, 2))
    if D_in != D:
        dq = dq[..., :D_in].contiguous()
        dk = dk.transpose(1, 2)[..., :D_in].contiguous().transpose(1, 2)
        dv = dv.transpose(1, 2)[..., :D_in].contiguous().transpose(1, 2)
    return dq, dk, dv
