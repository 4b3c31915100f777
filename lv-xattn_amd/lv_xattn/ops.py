"""One Python function per C entry point of liblvx.so, taking torch tensors.

These are the device operators the round loops in ``attn.py`` are made of; each
queues its kernel(s) on the current PyTorch stream and returns immediately.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import AttnShape, LvxError, check, load, ptr, stream_ptr, t4


@dataclass
class Mask:
    """Compact mask of a ragged / Llama-3.2-style batch.

    kv_len   int32 [B]      valid visual tokens per sample (None: all)
    kv_start int32 [B, Lq]  first visible visual token of each text row
    kv_end   int32 [B, Lq]  one past the last visible token (None: no interval mask)
    A row whose interval is empty sees nothing: O = 0, LSE = -inf, dQ = 0.
    """
    kv_len: Optional[torch.Tensor] = None
    kv_start: Optional[torch.Tensor] = None
    kv_end: Optional[torch.Tensor] = None

    def to(self, device) -> "Mask":
        f = lambda t: None if t is None else t.to(device=device, dtype=torch.int32).contiguous()
        return Mask(f(self.kv_len), f(self.kv_start), f(self.kv_end))


_DTYPES = {torch.bfloat16: _lib.LVX_BF16, torch.float16: _lib.LVX_F16}


def dtype_code(t: torch.Tensor, *others: torch.Tensor) -> int:
    """LVX_BF16 / LVX_F16 for the element type all the given tensors share."""
    if t.dtype not in _DTYPES or any(o.dtype != t.dtype for o in others):
        raise LvxError("bf16 or fp16 tensors of one type required, got "
                       + " / ".join(str(x.dtype) for x in (t,) + others))
    return _DTYPES[t.dtype]


def _shape(q: torch.Tensor, k: torch.Tensor, scale: float, mask: Optional[Mask],
           bias: Optional[torch.Tensor] = None) -> AttnShape:
    dt = dtype_code(q, k)
    B, Hq, Lq, D = q.shape
    Bk, Hkv, Lkv, Dk = k.shape
    if B != Bk or D != Dk:
        raise LvxError(f"q {tuple(q.shape)} and k {tuple(k.shape)} disagree on batch or head_dim")
    s = AttnShape(B, Hq, Hkv, D, Lq, Lkv, dt, float(scale), None, None, None)
    if mask is not None:
        for name in ("kv_len", "kv_start", "kv_end"):
            t = getattr(mask, name)
            if t is None:
                continue
            want = (B,) if name == "kv_len" else (B, Lq)
            if t.dtype != torch.int32 or tuple(t.shape) != want or not t.is_contiguous() or t.device != q.device:
                raise LvxError(f"mask.{name} must be a contiguous int32 {want} tensor on {q.device}")
            setattr(s, name, t.data_ptr())
    if bias is not None:
        if (bias.dtype != torch.float32 or bias.dim() != 4 or bias.device != q.device or bias.stride(3) != 1
                or bias.shape[0] not in (1, B) or bias.shape[1] not in (1, Hq) or tuple(bias.shape[2:]) != (Lq, Lkv)):
            raise LvxError(f"bias must be an fp32 [B|1, Hq|1, {Lq}, {Lkv}] tensor with unit last stride on {q.device}")
        # a dimension of extent 1 is never stepped over: whatever stride torch reports for it, the
        # library is told the value its own checks accept (0 to broadcast, the padded row length)
        row_stride = bias.stride(2) if Lq > 1 else (Lkv + 3) // 4 * 4
        if row_stride < (Lkv + 3) // 4 * 4:
            raise LvxError("bias rows must be padded to a multiple of 4 floats (row stride >= Lkv rounded up to 4)")
        if bias.data_ptr() % 16 or row_stride % 4 or any(bias.stride(i) % 4 and bias.shape[i] > 1 for i in range(2)):
            raise LvxError("bias must be 16-byte aligned with batch, head and row strides that are multiples of 4 floats")
        s.bias = bias.data_ptr()
        s.bias_stride_b = bias.stride(0) if bias.shape[0] > 1 else 0
        s.bias_stride_h = bias.stride(1) if bias.shape[1] > 1 else 0
        s.bias_stride_r = row_stride
    return s


def fwd_workspace_bytes(q, k, row_count: int, kv_splits: int) -> int:
    s = _shape(q, k, 1.0, None)
    return int(load().lvx_fwd_workspace_bytes(C.byref(s), row_count, kv_splits))


def fwd(q, k, v, o, lse, scale, row_begin=0, row_count=None, mask: Optional[Mask] = None,
        kv_splits: int = 1, workspace: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
        acc=None) -> None:
    """Partial O (bf16) and LSE (fp32 [B*Hq, Lq]) of text rows
    [row_begin, row_begin+row_count) against the whole local K/V shard.
    `bias`: dense additive fp32 [B|1, Hq|1, Lq, Lkv], added after the scale.
    `acc` = (o_in like o, l_in fp32 [B*Hq, Lq]): an incoming accumulator the result is merged
    with before it is written (lvx_fwd_acc); only read, and not o itself."""
    s = _shape(q, k, scale, mask, bias)
    if row_count is None:
        row_count = q.shape[2] - row_begin
    _check_lse(lse, q)
    ws_ptr, ws_bytes = (None, 0) if workspace is None else (workspace.data_ptr(), workspace.numel() * workspace.element_size())
    if acc is not None:
        o_in, l_in = acc
        dtype_code(q, o_in)
        _check_lse(l_in, q)
        rc = load().lvx_fwd_acc(C.byref(s), C.byref(t4(q)), C.byref(t4(k)), C.byref(t4(v)), C.byref(t4(o_in)),
                                l_in.data_ptr(), C.byref(t4(o)), lse.data_ptr(), row_begin, row_count, kv_splits,
                                ws_ptr, ws_bytes, stream_ptr())
        check(rc, "lvx_fwd_acc")
        return
    rc = load().lvx_fwd(C.byref(s), C.byref(t4(q)), C.byref(t4(k)), C.byref(t4(v)), C.byref(t4(o)),
                        lse.data_ptr(), row_begin, row_count, kv_splits, ws_ptr, ws_bytes, stream_ptr())
    check(rc, "lvx_fwd")


def noalloc_scratch_bytes() -> int:
    """Size of the library's own array that fwd_noalloc keeps its key-split partials in."""
    return int(load().lvx_noalloc_scratch_bytes())


def fwd_noalloc(q, k, v, o, lse, scale, row_begin=0, row_count=None, mask: Optional[Mask] = None,
                kv_splits: int = 1, bias: Optional[torch.Tensor] = None) -> None:
    """`fwd` without a workspace argument and without any allocation: the key-split
    partials go to an array inside the library (one per GPU, shared by all calls on it)."""
    s = _shape(q, k, scale, mask, bias)
    if row_count is None:
        row_count = q.shape[2] - row_begin
    _check_lse(lse, q)
    rc = load().lvx_fwd_noalloc(C.byref(s), C.byref(t4(q)), C.byref(t4(k)), C.byref(t4(v)), C.byref(t4(o)),
                                lse.data_ptr(), row_begin, row_count, kv_splits, stream_ptr())
    check(rc, "lvx_fwd_noalloc")


def merge(o_acc, l_acc, o_part, l_part, row_begin=0, row_count=None) -> None:
    """(o_acc, l_acc) <- LSE-merge of itself with (o_part, l_part), in place."""
    B, Hq, Lq, D = o_acc.shape
    s = AttnShape(B, Hq, Hq, D, Lq, 1, dtype_code(o_acc, o_part), 1.0, None, None, None)
    if row_count is None:
        row_count = Lq - row_begin
    _check_lse(l_acc, o_acc)
    _check_lse(l_part, o_acc)
    rc = load().lvx_merge(C.byref(s), C.byref(t4(o_acc)), l_acc.data_ptr(), C.byref(t4(o_part)),
                          l_part.data_ptr(), row_begin, row_count, stream_ptr())
    check(rc, "lvx_merge")


def bias_hull(q, k, bias: torch.Tensor) -> Mask:
    """The interval mask a dense bias implies: per text row the hull of its entries other
    than -inf.  Given to fwd / bwd together with the bias it lets them skip what the bias
    masks anyway."""
    s = _shape(q, k, 1.0, None, bias)
    B, Lq = q.shape[0], q.shape[2]
    start = torch.empty(B, Lq, dtype=torch.int32, device=q.device)
    end = torch.empty_like(start)
    rc = load().lvx_bias_hull(C.byref(s), start.data_ptr(), end.data_ptr(), stream_ptr())
    check(rc, "lvx_bias_hull")
    return Mask(None, start, end)


def bias_is_interval(q, k, bias: torch.Tensor, hull: Mask) -> bool:
    """Whether `bias` is nothing but the interval mask `hull` (from bias_hull): 0 wherever it is
    not -inf.  fwd / bwd with `hull` alone then give what they give with the bias, through the
    interval-mask kernels, which read no bias.  Waits for the GPU (one flag comes back)."""
    s = _shape(q, k, 1.0, None, bias)
    flag = torch.zeros(1, dtype=torch.int32, device=q.device)
    rc = load().lvx_bias_is_interval(C.byref(s), hull.kv_start.data_ptr(), hull.kv_end.data_ptr(), flag.data_ptr(),
                                     stream_ptr())
    check(rc, "lvx_bias_is_interval")
    return int(flag.item()) == 0


def bwd_preprocess(o, dout, delta, row_begin=0, row_count=None) -> None:
    B, Hq, Lq, D = o.shape
    s = AttnShape(B, Hq, Hq, D, Lq, 1, dtype_code(o, dout), 1.0, None, None, None)
    if row_count is None:
        row_count = Lq - row_begin
    _check_lse(delta, o)
    rc = load().lvx_bwd_preprocess(C.byref(s), C.byref(t4(o)), C.byref(t4(dout)), delta.data_ptr(),
                                   row_begin, row_count, stream_ptr())
    check(rc, "lvx_bwd_preprocess")


def bwd_workspace_bytes(q, k, row_count: int, mask: Optional[Mask] = None) -> int:
    """Bytes lvx_bwd needs for `row_count` rows; pass the mask the call will use
    (an interval mask adds its live-tile tables)."""
    s = _shape(q, k, 1.0, mask)
    return int(load().lvx_bwd_workspace_bytes(C.byref(s), row_count))


def bwd(q, k, v, dout, lse, delta, dq, dk, dv, scale, row_begin=0, row_count=None,
        mask: Optional[Mask] = None, accumulate_dkv: bool = False,
        workspace: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None) -> None:
    """Writes dq (bf16) for the selected rows and writes (bf16) or accumulates
    (fp32) dk, dv at Hkv heads.  `workspace`: uint8 tensor of at least
    bwd_workspace_bytes(q, k, row_count, mask) bytes.  `bias` as in fwd (no gradient
    is formed for it)."""
    s = _shape(q, k, scale, mask, bias)
    if row_count is None:
        row_count = q.shape[2] - row_begin
    _check_lse(lse, q)
    _check_lse(delta, q)
    if dq.dtype != q.dtype or dq.shape != q.shape:
        raise LvxError("dq must be a tensor of q's type and shape")
    want = torch.float32 if accumulate_dkv else q.dtype
    if dk.dtype != want or dv.dtype != want or dk.shape != k.shape or dv.shape != k.shape:
        raise LvxError(f"dk/dv must be {want} tensors shaped like k")
    if workspace is None:
        workspace = torch.empty(bwd_workspace_bytes(q, k, row_count, mask), dtype=torch.uint8, device=q.device)
    rc = load().lvx_bwd(C.byref(s), C.byref(t4(q)), C.byref(t4(k)), C.byref(t4(v)), C.byref(t4(dout)),
                        lse.data_ptr(), delta.data_ptr(), C.byref(t4(dq)), C.byref(t4(dk)), C.byref(t4(dv)),
                        1 if accumulate_dkv else 0, row_begin, row_count,
                        workspace.data_ptr(), workspace.numel() * workspace.element_size(), stream_ptr())
    check(rc, "lvx_bwd")


def cast_f32(src: torch.Tensor, dst: torch.Tensor) -> None:
    """dst (bf16 or fp16, [B,H,L,D] any strides) = src (fp32, memory order [B,H,L,D])."""
    B, H, L, D = dst.shape
    if src.dtype != torch.float32 or src.numel() != dst.numel():
        raise LvxError("cast_f32: fp32 source and 16-bit destination of equal size required")
    rc = load().lvx_cast_f32(src.data_ptr(), C.byref(t4(dst)), B, H, L, D, dtype_code(dst), stream_ptr())
    check(rc, "lvx_cast_f32")


def _rows2d(t: torch.Tensor, name: str) -> Tuple[int, int, int]:
    """[..., C] tensor whose leading dims collapse to rows with one stride."""
    if t.dtype not in _DTYPES:
        raise LvxError(f"{name}: bf16 or fp16 required")
    t2 = t.reshape(-1, t.shape[-1]) if t.is_contiguous() else None
    if t2 is None:
        raise LvxError(f"{name}: contiguous tensor required")
    return t2.data_ptr(), t2.shape[0], t2.stride(0)


def kv_proj(x_vis, w_k, w_v, n_kv_heads: int, w_in_major: bool = True,
            k_norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-5, for_backward: bool = False):
    """K, V = X W_k, X W_v.  x_vis [B, Lkv, Dm]; W [Dm, Hkv*D] (w_in_major) or
    [Hkv*D, Dm] (torch.nn.Linear.weight).  Returns [B, Hkv, Lkv, D] views of
    [B, Lkv, Hkv, D] memory.

    With `k_norm_weight` ([D] bf16) K is RMS-normalised per head in the GEMM's
    epilogue (the k_norm of test_llama3.py:418 in the reference).  With
    `for_backward` the call also returns what the norm's backward needs:
    (k, v, k_raw [B,Hkv,Lkv,D] view, k_rstd fp32 [B, Lkv, Hkv])."""
    B, Lkv, Dm = x_vis.shape
    N = w_k.shape[1] if w_in_major else w_k.shape[0]
    xp, M, ldx = _rows2d(x_vis, "x_vis")
    wkp, _, ldw = _rows2d(w_k, "w_k")
    wvp, _, ldw2 = _rows2d(w_v, "w_v")
    if ldw != ldw2 or w_k.shape != w_v.shape:
        raise LvxError("w_k and w_v must have the same shape")
    D = N // n_kv_heads
    dt = dtype_code(x_vis, w_k, w_v)
    k = torch.empty(B, Lkv, N, dtype=x_vis.dtype, device=x_vis.device)
    v = torch.empty_like(k)

    def heads(t):
        return t.view(B, Lkv, n_kv_heads, D).transpose(1, 2)

    if k_norm_weight is None:
        if for_backward:
            raise LvxError("for_backward only applies with k_norm_weight")
        rc = load().lvx_kv_proj(xp, ldx, wkp, wvp, ldw, 1 if w_in_major else 0, k.data_ptr(), v.data_ptr(), N,
                                M, Dm, N, dt, stream_ptr())
        check(rc, "lvx_kv_proj")
        return heads(k), heads(v)
    wn = _norm_weight(k_norm_weight, D, x_vis)
    k_raw = torch.empty_like(k) if for_backward else None
    rstd = torch.empty(B, Lkv, n_kv_heads, dtype=torch.float32, device=x_vis.device) if for_backward else None
    rc = load().lvx_kv_proj_norm(xp, ldx, wkp, wvp, ldw, 1 if w_in_major else 0, k.data_ptr(), v.data_ptr(), N,
                                 M, Dm, N, wn.data_ptr(), float(eps),
                                 k_raw.data_ptr() if for_backward else None,
                                 rstd.data_ptr() if for_backward else None, dt, stream_ptr())
    check(rc, "lvx_kv_proj_norm")
    if for_backward:
        return heads(k), heads(v), heads(k_raw), rstd
    return heads(k), heads(v)


def _norm_weight(w: torch.Tensor, D: int, like: torch.Tensor) -> torch.Tensor:
    if w.dtype != like.dtype or tuple(w.shape) != (D,) or D != 128:
        raise LvxError(f"the norm weight must be {like.dtype} [128], got {w.dtype} {tuple(w.shape)}")
    w = w.detach()
    if w.device != like.device:
        raise LvxError("k_norm_weight is on another device")
    if not w.is_contiguous() or w.data_ptr() % 16:
        w = w.contiguous().clone()
    return w


def k_norm_bwd(dk, k_raw, k_rstd, k_norm_weight, want_dw: bool = True):
    """Backward of the fused k_norm: returns (dk_raw, dw) with dk_raw a
    [B,Hkv,Lkv,D] view of new [B,Lkv,Hkv,D] memory and dw fp32 [D] (None
    unless `want_dw`)."""
    B, Hkv, Lkv, D = dk.shape
    dk2, kr2 = _token_major(dk, "dk"), _token_major(k_raw, "k_raw")
    N = Hkv * D
    wn = _norm_weight(k_norm_weight, D, dk)
    if k_rstd.dtype != torch.float32 or k_rstd.numel() != B * Lkv * Hkv or not k_rstd.is_contiguous():
        raise LvxError("k_rstd must be contiguous fp32 [B, Lkv, Hkv]")
    out = torch.empty(B, Lkv, N, dtype=dk.dtype, device=dk.device)
    dw = torch.zeros(D, dtype=torch.float32, device=dk.device) if want_dw else None
    rc = load().lvx_k_norm_bwd(dk2.data_ptr(), N, kr2.data_ptr(), N, k_rstd.data_ptr(), wn.data_ptr(),
                               out.data_ptr(), N, dw.data_ptr() if want_dw else None, B * Lkv, N,
                               dtype_code(dk, k_raw), stream_ptr())
    check(rc, "lvx_k_norm_bwd")
    return out.view(B, Lkv, Hkv, D).transpose(1, 2), dw


def q_proj(x, w_q, n_heads: int, w_in_major: bool = True, q_norm_weight: Optional[torch.Tensor] = None,
           eps: float = 1e-5, for_backward: bool = False):
    """Q = q_norm(X W_q) (test_llama3.py:390-393 in the reference): the K side of
    kv_proj on its own.  x [B, Lq, Dm]; returns a [B, Hq, Lq, D] view of
    [B, Lq, Hq, D] memory (and, with `for_backward`, the raw projection and r)."""
    B, Lq, Dm = x.shape
    N = w_q.shape[1] if w_in_major else w_q.shape[0]
    xp, M, ldx = _rows2d(x, "x")
    wp, _, ldw = _rows2d(w_q, "w_q")
    D = N // n_heads
    dt = dtype_code(x, w_q)
    q = torch.empty(B, Lq, N, dtype=x.dtype, device=x.device)

    def heads(t):
        return t.view(B, Lq, n_heads, D).transpose(1, 2)

    if q_norm_weight is None:
        if for_backward:
            raise LvxError("for_backward only applies with q_norm_weight")
        rc = load().lvx_kv_proj(xp, ldx, wp, None, ldw, 1 if w_in_major else 0, q.data_ptr(), None, N,
                                M, Dm, N, dt, stream_ptr())
        check(rc, "lvx_kv_proj")
        return heads(q)
    wn = _norm_weight(q_norm_weight, D, x)
    raw = torch.empty_like(q) if for_backward else None
    rstd = torch.empty(B, Lq, n_heads, dtype=torch.float32, device=x.device) if for_backward else None
    rc = load().lvx_kv_proj_norm(xp, ldx, wp, None, ldw, 1 if w_in_major else 0, q.data_ptr(), None, N,
                                 M, Dm, N, wn.data_ptr(), float(eps),
                                 raw.data_ptr() if for_backward else None,
                                 rstd.data_ptr() if for_backward else None, dt, stream_ptr())
    check(rc, "lvx_kv_proj_norm")
    if for_backward:
        return heads(q), heads(raw), rstd
    return heads(q)


def q_proj_bwd(x, dq_raw, w_q, w_in_major: bool = True, want_dw: bool = True):
    """(dX, dW_q) of Q_raw = X W_q from dq_raw ([B, Hq, Lq, D] view of
    [B, Lq, Hq, D] memory)."""
    B, Hq, Lq, D = dq_raw.shape
    N = Hq * D
    d2 = _token_major(dq_raw, "dq_raw")
    Dm = w_q.shape[0] if w_in_major else w_q.shape[1]
    wp, _, ldw = _rows2d(w_q, "w_q")
    xp, M, ldx = _rows2d(x, "x")
    dt = dtype_code(x, dq_raw, w_q)
    dx = torch.empty(B, Lq, Dm, dtype=x.dtype, device=x.device)
    rc = load().lvx_dx_vis(d2.data_ptr(), None, N, wp, None, ldw, 1 if w_in_major else 0, dx.data_ptr(), Dm,
                           M, Dm, N, dt, stream_ptr())
    check(rc, "lvx_dx_vis")
    dw = None
    if want_dw:
        shape = (Dm, N) if w_in_major else (N, Dm)
        dw = torch.empty(*shape, dtype=x.dtype, device=x.device)
        rc = load().lvx_dw_kv(xp, ldx, d2.data_ptr(), None, N, dw.data_ptr(), None, shape[1],
                              1 if w_in_major else 0, M, Dm, N, dt, stream_ptr())
        check(rc, "lvx_dw_kv")
    return dx, dw


def _token_major(t: torch.Tensor, name: str) -> torch.Tensor:
    """[B, Hkv, Lkv, D] view whose memory is [B, Lkv, Hkv, D] -> [B*Lkv, Hkv*D]."""
    tm = t.transpose(1, 2)
    if not tm.is_contiguous():
        raise LvxError(f"{name} must be a [B,Hkv,Lkv,D] view of contiguous [B,Lkv,Hkv,D] memory")
    return tm.reshape(tm.shape[0] * tm.shape[1], -1)


def dx_vis(dk, dv, w_k, w_v, w_in_major: bool = True) -> torch.Tensor:
    """dX = dK W_k^T + dV W_v^T -> [B, Lkv, Dm]."""
    B, Hkv, Lkv, D = dk.shape
    dk2, dv2 = _token_major(dk, "dk"), _token_major(dv, "dv")
    N = Hkv * D
    Dm = w_k.shape[0] if w_in_major else w_k.shape[1]
    wkp, _, ldw = _rows2d(w_k, "w_k")
    wvp, _, _ = _rows2d(w_v, "w_v")
    dx = torch.empty(B, Lkv, Dm, dtype=dk.dtype, device=dk.device)
    rc = load().lvx_dx_vis(dk2.data_ptr(), dv2.data_ptr(), N, wkp, wvp, ldw, 1 if w_in_major else 0,
                           dx.data_ptr(), Dm, B * Lkv, Dm, N, dtype_code(dk, dv, w_k, w_v), stream_ptr())
    check(rc, "lvx_dx_vis")
    return dx


def dw_kv(x_vis, dk, dv, w_in_major: bool = True):
    """dW_k = X^T dK, dW_v = X^T dV in the layout of W."""
    B, Lkv, Dm = x_vis.shape
    Hkv, D = dk.shape[1], dk.shape[3]
    N = Hkv * D
    dk2, dv2 = _token_major(dk, "dk"), _token_major(dv, "dv")
    xp, M, ldx = _rows2d(x_vis, "x_vis")
    shape = (Dm, N) if w_in_major else (N, Dm)
    dwk = torch.empty(*shape, dtype=x_vis.dtype, device=x_vis.device)
    dwv = torch.empty_like(dwk)
    rc = load().lvx_dw_kv(xp, ldx, dk2.data_ptr(), dv2.data_ptr(), N, dwk.data_ptr(), dwv.data_ptr(), shape[1],
                          1 if w_in_major else 0, M, Dm, N, dtype_code(x_vis, dk, dv), stream_ptr())
    check(rc, "lvx_dw_kv")
    return dwk, dwv


def _check_lse(l: torch.Tensor, q: torch.Tensor) -> None:
    B, Hq, Lq, _ = q.shape
    if l.dtype != torch.float32 or not l.is_contiguous() or l.numel() != B * Hq * Lq:
        raise LvxError(f"LSE/delta must be contiguous fp32 with {B * Hq * Lq} elements ([B*Hq, Lq])")
