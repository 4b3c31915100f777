"""lvx_fwd_noalloc - the forward entry point whose key-split partials live in an array inside
the library instead of a caller's workspace - against lvx_fwd on the same inputs, through the
C ABI: two calls in a row, the second on a smaller input (the array keeps the first call's
contents), bit for bit, and against the CPU oracle; then the size limit."""
import ctypes as C

import pytest
import torch

from oracle import lvx_oracle as orc
from parity import check_lse, check_o

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(B, Hq, Hkv, Lq, Lkv, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, Lq, 128, generator=g).bfloat16().to(DEV)
    k = torch.randn(B, Hkv, Lkv, 128, generator=g).bfloat16().to(DEV)
    v = torch.randn(B, Hkv, Lkv, 128, generator=g).bfloat16().to(DEV)
    return q, k, v


def _both(ops, q, k, v, splits, row_begin, row_count):
    B, Hq, Lq, _ = q.shape
    scale = 128 ** -0.5
    o_ref = torch.zeros_like(q)
    l_ref = torch.zeros(B * Hq, Lq, device=DEV)
    ws = torch.empty(ops.fwd_workspace_bytes(q, k, row_count, splits), dtype=torch.uint8, device=DEV)
    ops.fwd(q, k, v, o_ref, l_ref, scale, row_begin, row_count, None, splits, ws)
    o = torch.zeros_like(q)
    l = torch.zeros(B * Hq, Lq, device=DEV)
    ops.fwd_noalloc(q, k, v, o, l, scale, row_begin, row_count, None, splits)
    torch.cuda.synchronize()
    return o, l, o_ref, l_ref


def test_noalloc_forward_matches_forward_twice_then_rejects_what_does_not_fit():
    from lv_xattn import _lib, ops
    lib = _lib.load()
    assert ops.noalloc_scratch_bytes() == 16 << 20

    # first call: 4 key splits over 1000 keys, a 200-row window of 256 rows (fills 6.6 MB of the array)
    q, k, v = _inputs(1, 32, 8, 256, 1000, 11)
    assert ops.fwd_workspace_bytes(q, k, 200, 4) <= ops.noalloc_scratch_bytes()
    o, l, o_ref, l_ref = _both(ops, q, k, v, 4, 30, 200)
    assert torch.equal(o, o_ref) and torch.equal(l, l_ref)
    assert o[:, :, 30:230].abs().max() > 0

    # second call, smaller in every size: the array still holds the partials of the first
    q2, k2, v2 = _inputs(2, 8, 2, 96, 700, 12)
    o, l, o_ref, l_ref = _both(ops, q2, k2, v2, 2, 0, 96)
    assert torch.equal(o, o_ref) and torch.equal(l, l_ref)
    assert o.abs().max() > 0
    # and on its own feet: the second call against the CPU oracle (full softmax in fp32)
    o_orc, l_orc = orc.attention_dense(q2.float().cpu(), k2.float().cpu(), v2.float().cpu(), 128 ** -0.5)
    check_o(o, o_orc, "O of lvx_fwd_noalloc")
    check_lse(l, l_orc, "LSE of lvx_fwd_noalloc")

    # one split needs no array at all
    o, l, o_ref, l_ref = _both(ops, q, k, v, 1, 0, 256)
    assert torch.equal(o, o_ref) and torch.equal(l, l_ref)

    # partials beyond the array: rejected on the host, nothing launched, outputs untouched
    qb, kb, vb = _inputs(1, 32, 8, 4096, 1024, 13)
    assert ops.fwd_workspace_bytes(qb, kb, 4096, 2) > ops.noalloc_scratch_bytes()
    ob = torch.full_like(qb, 7.0)
    lb = torch.full((32, 4096), 7.0, device=DEV)
    s = ops._shape(qb, kb, 128 ** -0.5, None)
    rc = lib.lvx_fwd_noalloc(C.byref(s), C.byref(_lib.t4(qb)), C.byref(_lib.t4(kb)), C.byref(_lib.t4(vb)),
                             C.byref(_lib.t4(ob)), lb.data_ptr(), 0, 4096, 2, _lib.stream_ptr())
    torch.cuda.synchronize()
    assert rc == -7 and b"workspace" in lib.lvx_strerror(rc)
    assert bool((ob == 7.0).all()) and bool((lb == 7.0).all())
