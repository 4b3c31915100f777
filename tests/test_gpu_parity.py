"""GPU parity tests: the HIP path, called through the C ABI, against the CPU
oracle on the same seeded inputs.  Tolerances: O max-abs <= 2e-2 and mean-abs
<= 2e-3, LSE <= 1e-3 abs (-inf exactly for rows that see nothing), gradients
the same bounds scaled by max|ref| plus relative L2 <= 1e-2."""
import math

import pytest
import torch

from oracle import lvx_oracle as orc
from parity import check_grad, check_lse, check_o

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def lvx():
    import lv_xattn
    from lv_xattn import _lib
    _lib.load()
    return lv_xattn


def _dev(t):
    return t.to(DEV)


def _mask_of(w, lvx):
    t = w.tensors
    kv_len = torch.tensor(w.kv_len, dtype=torch.int32) if w.kv_len else None
    if "kv_start" in t or kv_len is not None:
        return lvx.Mask(kv_len, t.get("kv_start"), t.get("kv_end"))
    return None


# ------------------------------------------------------------------ GEMMs
@pytest.mark.parametrize("w_in_major", [True, False])
def test_kv_proj_dx_dw_small(lvx, w_in_major):
    from lv_xattn import ops
    g = torch.Generator().manual_seed(5)
    B, L, Dm, Hkv, D = 2, 333, 328, 2, 128          # ragged rows, Dm not a multiple of 64
    x = (torch.randn(B, L, Dm, generator=g) * 0.5).bfloat16()
    wk = (torch.randn(Dm, Hkv * D, generator=g) * 0.1).bfloat16()
    wv = (torch.randn(Dm, Hkv * D, generator=g) * 0.1).bfloat16()
    k_ref, v_ref = orc.kv_project(x, wk, wv, Hkv)
    wk_d, wv_d = (wk, wv) if w_in_major else (wk.t().contiguous(), wv.t().contiguous())
    k, v = ops.kv_proj(_dev(x), _dev(wk_d), _dev(wv_d), Hkv, w_in_major)
    torch.cuda.synchronize()
    check_grad(k, k_ref, "K")
    check_grad(v, v_ref, "V")
    assert k.transpose(1, 2).is_contiguous()

    dk = (torch.randn(B, L, Hkv, D, generator=g)).bfloat16().transpose(1, 2)
    dv = (torch.randn(B, L, Hkv, D, generator=g)).bfloat16().transpose(1, 2)
    dx_ref = orc.dx_vis(dk, dv, wk, wv)
    dx = ops.dx_vis(_dev(dk.transpose(1, 2).contiguous()).transpose(1, 2),
                    _dev(dv.transpose(1, 2).contiguous()).transpose(1, 2), _dev(wk_d), _dev(wv_d), w_in_major)
    torch.cuda.synchronize()
    check_grad(dx, dx_ref, "dX_vis")

    dwk_ref, dwv_ref = orc.dw_kv(x, dk, dv)
    dwk, dwv = ops.dw_kv(_dev(x), _dev(dk.transpose(1, 2).contiguous()).transpose(1, 2),
                         _dev(dv.transpose(1, 2).contiguous()).transpose(1, 2), w_in_major)
    torch.cuda.synchronize()
    if not w_in_major:
        dwk, dwv = dwk.t(), dwv.t()
    check_grad(dwk, dwk_ref, "dW_k")
    check_grad(dwv, dwv_ref, "dW_v")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w_in_major", [True, False])
def test_kv_proj_fused_k_norm_and_its_backward(lvx, w_in_major, dtype):
    from lv_xattn import ops
    g = torch.Generator().manual_seed(6)
    B, L, Dm, Hkv, D = 2, 301, 264, 4, 128          # ragged rows; 512 columns = two column tiles
    x = (torch.randn(B, L, Dm, generator=g) * 0.5).to(dtype)
    wk = (torch.randn(Dm, Hkv * D, generator=g) * 0.1).to(dtype)
    wv = (torch.randn(Dm, Hkv * D, generator=g) * 0.1).to(dtype)
    wn = (1.0 + 0.3 * torch.randn(D, generator=g)).to(dtype)
    eps = 1e-5
    k_raw_ref, v_ref = orc.kv_project(x, wk, wv, Hkv)
    k_raw_ref = k_raw_ref.to(dtype)
    k_ref = orc.k_rms_norm(k_raw_ref, wn, eps)
    wk_d, wv_d = (wk, wv) if w_in_major else (wk.t().contiguous(), wv.t().contiguous())
    k, v, k_raw, rstd = ops.kv_proj(_dev(x), _dev(wk_d), _dev(wv_d), Hkv, w_in_major, k_norm_weight=_dev(wn),
                                    eps=eps, for_backward=True)
    k2, v2 = ops.kv_proj(_dev(x), _dev(wk_d), _dev(wv_d), Hkv, w_in_major, k_norm_weight=_dev(wn), eps=eps)
    torch.cuda.synchronize()
    check_grad(k, k_ref, "K (normed)")
    check_grad(v, v_ref, "V")
    check_grad(k_raw, k_raw_ref, "K (raw)")
    assert torch.equal(k, k2) and torch.equal(v, v2)          # the optional outputs change nothing
    r_ref = torch.rsqrt(k_raw_ref.float().pow(2).mean(-1) + eps).transpose(1, 2)     # [B, L, Hkv]
    assert tuple(rstd.shape) == (B, L, Hkv)
    assert ((rstd.cpu() - r_ref).abs() <= 1e-2 * r_ref).all()

    dk = torch.randn(B, L, Hkv, D, generator=g).to(dtype).transpose(1, 2)
    dx_ref, dw_ref = orc.k_rms_norm_backward(dk, k_raw.float().cpu(), wn, eps)
    dk_raw, dw = ops.k_norm_bwd(_dev(dk.transpose(1, 2).contiguous()).transpose(1, 2), k_raw, rstd, _dev(wn))
    torch.cuda.synchronize()
    check_grad(dk_raw, dx_ref, "dK (raw)")
    check_grad(dw, dw_ref, "dw_norm")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w_in_major", [True, False])
def test_q_projection_with_q_norm_autograd(lvx, w_in_major, dtype):
    # the text side of `project`: Q = q_norm(X W_q), recomputed in backward
    g = torch.Generator().manual_seed(8)
    B, L, Dm, Hq, D = 2, 203, 328, 3, 128
    x = (torch.randn(B, L, Dm, generator=g) * 0.5).to(dtype)
    wq = (torch.randn(Dm, Hq * D, generator=g) * 0.1).to(dtype)
    wn = (1.0 + 0.3 * torch.randn(D, generator=g)).to(dtype)
    dq = torch.randn(B, Hq, L, D, generator=g).to(dtype)
    q_raw_ref, _ = orc.kv_project(x, wq, wq, Hq)
    q_raw_ref = q_raw_ref.to(dtype)
    q_ref = orc.k_rms_norm(q_raw_ref, wn, 1e-5)
    dq_raw_ref, dwn_ref = orc.k_rms_norm_backward(dq, q_raw_ref, wn, 1e-5)
    dx_ref = orc.dx_vis(dq_raw_ref.to(dtype), torch.zeros_like(dq_raw_ref), wq, wq)
    dw_ref, _ = orc.dw_kv(x, dq_raw_ref.to(dtype), torch.zeros_like(dq_raw_ref))

    proj = lvx.create_q_projection_class(w_in_major=w_in_major).apply
    xd = _dev(x).requires_grad_()
    wd = _dev(wq if w_in_major else wq.t().contiguous()).requires_grad_()
    wnd = _dev(wn).requires_grad_()
    q = proj(xd, wd, Hq, wnd, 1e-5)
    assert tuple(q.shape) == (B, Hq, L, D)
    q.backward(_dev(dq))
    torch.cuda.synchronize()
    check_grad(q.detach(), q_ref, "Q")
    check_grad(xd.grad, dx_ref, "dX")
    check_grad(wd.grad if w_in_major else wd.grad.t(), dw_ref, "dW_q")
    check_grad(wnd.grad, dwn_ref, "dw_norm")


def test_reference_call_shape_of_the_recompute_wrapper(lvx):
    """attention(hidden_states, project, is_causal) exactly as the reference's patched forward calls
    it (test_llama3.py:184-243, 459): q, k, v come from run_function(x, global visual states) in
    both passes, only (x, o, L) are kept, and - unlike the reference (:243) - every input of the
    projection gets its gradient.  Checked against the oracle's layer (projection with q_norm /
    k_norm, attention, backward through all of it)."""
    g = torch.Generator().manual_seed(21)
    B, Lq, Lkv, Dm, Hq, Hkv, D = 2, 96, 301, 256, 8, 2, 128
    dt = torch.bfloat16
    x = (torch.randn(B, Lq, Dm, generator=g) * 0.5).to(dt)
    vis = (torch.randn(B, Lkv, Dm, generator=g) * 0.5).to(dt)
    wq = (torch.randn(Dm, Hq * D, generator=g) * 0.08).to(dt)
    wk = (torch.randn(Dm, Hkv * D, generator=g) * 0.08).to(dt)
    wv = (torch.randn(Dm, Hkv * D, generator=g) * 0.08).to(dt)
    wqn = (1.0 + 0.2 * torch.randn(D, generator=g)).to(dt)
    wkn = (1.0 + 0.2 * torch.randn(D, generator=g)).to(dt)
    do = torch.randn(B, Hq, Lq, D, generator=g).to(dt)
    scale = D ** -0.5
    # oracle: projections (rounded to bf16 where the device stores them), norms, attention, all the way back
    q_raw, _ = orc.kv_project(x, wq, wq, Hq)
    q_raw = q_raw.to(dt)
    q_ref = orc.k_rms_norm(q_raw, wqn, 1e-5).to(dt)
    k_raw, v_ref = orc.kv_project(vis, wk, wv, Hkv)
    k_raw, v_ref = k_raw.to(dt), v_ref.to(dt)
    k_ref = orc.k_rms_norm(k_raw, wkn, 1e-5).to(dt)
    o_ref, l_ref = orc.round_loop_forward(q_ref, k_ref, v_ref, scale, 1)
    dq_ref, dk_ref, dv_ref = orc.attention_backward(do, q_ref, k_ref, v_ref, o_ref, l_ref, scale)
    dq_raw_ref, dwqn_ref = orc.k_rms_norm_backward(dq_ref.to(dt), q_raw, wqn, 1e-5)
    dk_raw_ref, dwkn_ref = orc.k_rms_norm_backward(dk_ref.to(dt), k_raw, wkn, 1e-5)
    dx_ref = orc.dx_vis(dq_raw_ref.to(dt), torch.zeros_like(dq_raw_ref), wq, wq)
    dvis_ref = orc.dx_vis(dk_raw_ref.to(dt), dv_ref.to(dt), wk, wv)
    dwq_ref, _ = orc.dw_kv(x, dq_raw_ref.to(dt), torch.zeros_like(dq_raw_ref))
    dwk_ref, dwv_ref = orc.dw_kv(vis, dk_raw_ref.to(dt), dv_ref.to(dt))

    xd, visd = _dev(x).requires_grad_(), _dev(vis).requires_grad_()
    wqd, wkd, wvd = (_dev(t).requires_grad_() for t in (wq, wk, wv))
    wqnd, wknd = _dev(wqn).requires_grad_(), _dev(wkn).requires_grad_()
    q_proj, kv_proj = lvx.create_q_projection_class().apply, lvx.create_kv_projection_class().apply
    calls = []

    def project(hidden_states, cross_attention_states):      # the reference's closure, on this library's GEMMs
        calls.append(torch.is_grad_enabled())
        query_states = q_proj(hidden_states, wqd, Hq, wqnd, 1e-5)
        key_states, value_states = kv_proj(cross_attention_states, wkd, wvd, Hkv, wknd, 1e-5)
        return query_states, key_states, value_states

    attention = lvx.create_attention_class("lv_xattn", no_overlap=False).apply
    lvx.set_global_cross_attention_states(visd)
    try:
        o = attention(xd, project, False)
        assert len(o.grad_fn.saved_tensors) == 3        # x, o, L: neither Q nor K nor V is kept
        o.backward(_dev(do))
        torch.cuda.synchronize()
    finally:
        lvx.clear_global_cross_attention_states()
    assert calls == [False, True]                        # forward without a graph, backward's recompute with one
    check_o(o.detach(), o_ref)
    check_grad(xd.grad, dx_ref, "dX")
    check_grad(visd.grad, dvis_ref, "dX_vis")
    check_grad(wqd.grad, dwq_ref, "dW_q")
    check_grad(wkd.grad, dwk_ref, "dW_k")
    check_grad(wvd.grad, dwv_ref, "dW_v")
    check_grad(wqnd.grad, dwqn_ref, "dw_q_norm")
    check_grad(wknd.grad, dwkn_ref, "dw_k_norm")
    with pytest.raises(ValueError, match=r"test_llama3\.py:430"):
        attention(xd, project, True)


# ------------------------------------------------------------------ row-wise kernels
def test_merge_ignores_an_accumulator_that_holds_nothing_yet(lvx):
    """(garbage, L = -inf) is the identity of the merge: a travelling accumulator may start as
    uninitialised memory with L = -inf, whatever bits its O holds."""
    from lv_xattn import ops
    g = torch.Generator().manual_seed(9)
    B, H, L, D = 1, 2, 40, 128
    ob = torch.randn(B, H, L, D, generator=g).bfloat16()
    lb = torch.randn(B, H, L, generator=g) + 5
    lb[0, 1, 7] = float("-inf")                         # a part that saw no key either
    o_acc = torch.full((B, H, L, D), float("nan")).bfloat16()
    o_acc[0, 0, 1] = float("inf")
    l_acc = torch.full((B * H, L), float("-inf"))
    o_d, l_d = _dev(o_acc), _dev(l_acc)
    ops.merge(o_d, l_d, _dev(ob), _dev(lb).reshape(B * H, L).contiguous())
    torch.cuda.synchronize()
    want = ob.clone()
    want[0, 1, 7] = 0
    assert torch.equal(o_d.cpu(), want)
    assert torch.equal(l_d.cpu(), lb.reshape(B * H, L))


def test_merge_against_oracle(lvx):
    from lv_xattn import ops
    g = torch.Generator().manual_seed(7)
    B, H, L, D = 2, 3, 77, 128
    oa = torch.randn(B, H, L, D, generator=g).bfloat16()
    ob = torch.randn(B, H, L, D, generator=g).bfloat16()
    la = torch.randn(B, H, L, generator=g) * 3 + 9
    lb = torch.randn(B, H, L, generator=g) * 3 + 9
    la[0, 0, :5] = float("-inf")
    lb[0, 0, 3:9] = float("-inf")
    la[1, 2, 10] = 300.0          # would overflow a naive exp()
    o_ref, l_ref = orc.merge_lse(oa.float(), la, ob.float(), lb)
    o_d, l_d = _dev(oa).clone(), _dev(la).reshape(B * H, L).clone()
    ops.merge(o_d, l_d, _dev(ob), _dev(lb).reshape(B * H, L).contiguous())
    torch.cuda.synchronize()
    check_o(o_d, o_ref, "merged O")
    check_lse(l_d, l_ref, "merged LSE")
    # row window: rows outside stay untouched
    o_d2, l_d2 = _dev(oa).clone(), _dev(la).reshape(B * H, L).clone()
    ops.merge(o_d2, l_d2, _dev(ob), _dev(lb).reshape(B * H, L).contiguous(), 16, 20)
    torch.cuda.synchronize()
    assert torch.equal(o_d2[:, :, :16].cpu(), oa[:, :, :16]) and torch.equal(o_d2[:, :, 36:].cpu(), oa[:, :, 36:])
    assert torch.equal(o_d2[:, :, 16:36], o_d[:, :, 16:36])


def test_preprocess_delta(lvx):
    from lv_xattn import ops
    g = torch.Generator().manual_seed(8)
    B, H, L, D = 1, 5, 61, 128
    o = torch.randn(B, H, L, D, generator=g).bfloat16()
    do = torch.randn(B, H, L, D, generator=g).bfloat16()
    delta = torch.zeros(B * H, L, device=DEV)
    ops.bwd_preprocess(_dev(o), _dev(do), delta)
    torch.cuda.synchronize()
    ref = orc.bwd_delta(o, do).reshape(B * H, L)
    assert (delta.cpu() - ref).abs().max() < 1e-3


# ------------------------------------------------------------------ forward
@pytest.fixture(params=["auto", "wide"])
def form(request, monkeypatch):
    """The bf16 forward kernel for launches without interval mask or bias has two forms: a wave owns 32
    rows, or 64 rows and its SIMD (picked when every CU gets a work-group).  'wide' forces the second
    on these small shapes - also with ragged row counts, ragged key lengths, key splits and incoming
    accumulators - through the environment variable the library reads at every call (masked launches
    take the plain kernel either way)."""
    if request.param == "wide":
        monkeypatch.setenv("LVX_FWD_WIDE", "1")
    return request.param


@pytest.mark.parametrize("mode", ["rounds", "batched", "splits"])
def test_forward_cfg1s(lvx, mode, form):
    w = orc.make_inputs(orc.workload("cfg1s"))
    t = w.tensors
    o_ref, l_ref = orc.round_loop_forward(t["q"], t["k"], t["v"], w.scale, w.rounds)
    kw = dict(rounds=w.rounds)
    if mode == "batched":
        kw["batched"] = True
    if mode == "splits":
        kw["kv_splits"] = 4
    _, _, _, o, L = lvx._attn_forward(_dev(t["q"]), _dev(t["k"]), _dev(t["v"]), False, w.scale, None, **kw)
    torch.cuda.synchronize()
    assert o.dtype == torch.bfloat16 and L.shape == (w.B * w.Hq, w.Lq) and L.dtype == torch.float32
    check_o(o, o_ref)
    check_lse(L, l_ref)


@pytest.mark.parametrize("kw", [dict(), dict(kv_splits=1), dict(kv_splits=4), dict(batched=True),
                                dict(batched=True, kv_splits=3)],
                         ids=["auto", "nosplit", "split4", "batched", "batched_split3"])
def test_forward_with_incoming_accumulator(lvx, kw, form):
    # lvx_fwd_acc: the round's partial and the travelling accumulator leave as one result; with
    # key splits one merge launch folds the splits and the accumulator, which may hold NaN
    # where its LSE is -inf (nothing folded in yet)
    w = orc.make_inputs(orc.workload("cfg1s"))
    t = w.tensors
    g = torch.Generator().manual_seed(11)
    o_in = torch.randn(w.B, w.Hq, w.Lq, w.D, generator=g).bfloat16()
    l_in = torch.randn(w.B, w.Hq, w.Lq, generator=g) * 0.1 + math.log(w.Lkv) + 0.5
    l_in[:, :, 5::17] = float("-inf")
    o_clean = o_in.clone()
    o_clean[l_in.isinf()] = 0
    o_in[l_in.isinf()] = float("nan")
    o_ref, l_ref = orc.round_loop_forward(t["q"], t["k"], t["v"], w.scale, w.rounds,
                                          acc_in=(o_clean, l_in), round_to_bf16=True)
    o_d, l_d = _dev(o_in), _dev(l_in)
    _, _, _, o, L = lvx._attn_forward(_dev(t["q"]), _dev(t["k"]), _dev(t["v"]), False, w.scale, None,
                                      rounds=w.rounds, acc_in=(o_d, l_d), **kw)
    torch.cuda.synchronize()
    check_o(o, o_ref)
    check_lse(L, l_ref)
    # the accumulator is only read
    assert torch.equal(l_d.cpu(), l_in) and torch.equal(o_d.cpu().isnan(), o_in.isnan())


def test_forward_kv_chunks_then_merge_equals_full_softmax(lvx):
    # one query block visiting 4 "GPUs": partial per 401-token chunk + sequential merge
    from lv_xattn import ops
    w = orc.make_inputs(orc.workload("cfg1s"))
    t = w.tensors
    o_ref, l_ref = orc.attention_dense(t["q"], t["k"], t["v"], w.scale)
    q, k, v = _dev(t["q"]), _dev(t["k"]), _dev(t["v"])
    o_acc = torch.zeros_like(q)
    l_acc = torch.full((w.B * w.Hq, w.Lq), float("-inf"), device=DEV)
    o_p, l_p = torch.empty_like(q), torch.empty_like(l_acc)
    for c0 in range(0, w.Lkv, 401):
        c1 = min(c0 + 401, w.Lkv)
        ops.fwd(q, k[:, :, c0:c1], v[:, :, c0:c1], o_p, l_p, w.scale)
        ops.merge(o_acc, l_acc, o_p, l_p)
    torch.cuda.synchronize()
    check_o(o_acc, o_ref)
    check_lse(l_acc, l_ref)


def test_forward_masked_ragged_cfg4s(lvx, form):
    w = orc.make_inputs(orc.workload("cfg4s"))
    t = w.tensors
    allowed = orc.workload_allowed(w)
    o_ref, l_ref = orc.round_loop_forward(t["q"], t["k"], t["v"], w.scale, w.rounds, allowed=allowed)
    for kw in (dict(), dict(batched=True), dict(kv_splits=3)):
        _, _, _, o, L = lvx._attn_forward(_dev(t["q"]), _dev(t["k"]), _dev(t["v"]), False, w.scale, None,
                                          rounds=w.rounds, mask=_mask_of(w, lvx), **kw)
        torch.cuda.synchronize()
        check_o(o, o_ref, f"O {kw}")
        check_lse(L, l_ref, f"LSE {kw}")
        dead = torch.isinf(l_ref)
        assert (o.float().cpu()[dead] == 0).all()


def test_forward_kv_len_only(lvx, form):
    w = orc.make_inputs(orc.workload("cfg4s"))
    t = w.tensors
    w.tensors = {k_: v_ for k_, v_ in t.items() if not k_.startswith("kv_")}
    allowed = orc.workload_allowed(w)
    o_ref, l_ref = orc.attention_dense(t["q"], t["k"], t["v"], w.scale, allowed=allowed)
    mask = lvx.Mask(torch.tensor(w.kv_len, dtype=torch.int32))
    _, _, _, o, L = lvx._attn_forward(_dev(t["q"]), _dev(t["k"]), _dev(t["v"]), False, w.scale, None,
                                      rounds=1, mask=mask)
    torch.cuda.synchronize()
    check_o(o, o_ref)
    check_lse(L, l_ref)


def test_forward_mha_and_gqa8_strided_inputs(lvx, form):
    # G = 1 (one head x 128 rows per work-group) and G = 8 (two groups per kv head);
    # q/k/v given as [B,S,H,D]-memory views, as a fused projection would produce them
    g = torch.Generator().manual_seed(21)
    for Hq, Hkv in ((3, 3), (8, 1)):
        q = torch.randn(1, 200, Hq, 128, generator=g).bfloat16().transpose(1, 2)
        k = torch.randn(1, 300, Hkv, 128, generator=g).bfloat16().transpose(1, 2)
        v = torch.randn(1, 300, Hkv, 128, generator=g).bfloat16().transpose(1, 2)
        o_ref, l_ref = orc.attention_dense(q, k, v, 0.11)
        _, _, _, o, L = lvx._attn_forward(_dev(q), _dev(k), _dev(v), False, 0.11, None, rounds=3)
        torch.cuda.synchronize()
        check_o(o, o_ref, f"O Hq{Hq} Hkv{Hkv}")
        check_lse(L, l_ref, f"LSE Hq{Hq} Hkv{Hkv}")


# ------------------------------------------------------------------ backward
@pytest.mark.parametrize("batched", [False, True])
def test_backward_cfg1s(lvx, batched):
    w = orc.make_inputs(orc.workload("cfg1s"))
    t = w.tensors
    ref = orc.layer_reference(w)
    q, k, v, do = (_dev(t[n]) for n in ("q", "k", "v", "do"))
    _, _, _, o, L = lvx._attn_forward(q, k, v, False, w.scale, None, rounds=w.rounds, batched=batched)
    dq, dk, dv = lvx._attn_backward(do, q, k, v, o, L, False, w.scale, None, "flash",
                                    rounds=w.rounds, batched=batched)
    torch.cuda.synchronize()
    assert dk.shape == k.shape and dv.shape == v.shape and dq.shape == q.shape
    check_grad(dq, ref["dq"], "dQ")
    check_grad(dk, ref["dk"], "dK")
    check_grad(dv, ref["dv"], "dV")


@pytest.mark.parametrize("name", ["cfg1s", "cfg4s"])
def test_rounds_spread_over_streams(lvx, name):
    """The rounds of a call touch disjoint rows; queued on three streams instead of one they give
    the same O, LSE and dQ bit for bit, and dK / dV up to the order of the fp32 sums."""
    w = orc.make_inputs(orc.workload(name))
    t = w.tensors
    ref = orc.layer_reference(w)
    q, k, v, do = (_dev(t[n]) for n in ("q", "k", "v", "do"))
    mask = _mask_of(w, lvx)
    acc = (torch.zeros_like(q), torch.full((w.B * w.Hq, w.Lq), float("-inf"), device=DEV))
    res = []
    for n in (1, 3):
        _, _, _, o, L = lvx._attn_forward(q, k, v, False, w.scale, None, rounds=w.rounds, mask=mask, acc_in=acc,
                                          streams=n)
        dq, dk, dv = lvx._attn_backward(do, q, k, v, o, L, False, w.scale, None, "flash", rounds=w.rounds, mask=mask,
                                        streams=n)
        torch.cuda.synchronize()
        res.append((o, L, dq, dk, dv))
    (o1, l1, dq1, dk1, dv1), (o3, l3, dq3, dk3, dv3) = res
    assert torch.equal(o1, o3) and torch.equal(l1, l3) and torch.equal(dq1, dq3)
    check_o(o3, ref["o"])
    check_lse(l3, ref["lse"])
    check_grad(dq3, ref["dq"], "dQ")
    check_grad(dk3, ref["dk"], "dK")
    check_grad(dv3, ref["dv"], "dV")
    for a, b_ in ((dk1, dk3), (dv1, dv3)):
        assert (a.float() - b_.float()).abs().max() <= 1e-2 * a.float().abs().max()


def test_backward_in_row_chunks_under_a_small_workspace_cap(lvx):
    """A window whose dS^T workspace would exceed the cap runs as several calls over row chunks
    (fp32 dK / dV across them): same gradients as the single call."""
    from lv_xattn import async_communication as ac
    w = orc.workload("cfg1s")
    w.Lq, w.rounds = 1024, 1
    w = orc.make_inputs(w)
    t = w.tensors
    ref = orc.layer_reference(w)
    q, k, v, do = (_dev(t[n]) for n in ("q", "k", "v", "do"))
    _, _, _, o, L = lvx._attn_forward(q, k, v, False, w.scale, None, rounds=1, batched=True)
    one = lvx._attn_backward(do, q, k, v, o, L, False, w.scale, None, "flash", rounds=1, batched=True)
    old = ac.backward_workspace_cap()
    seen = []
    real = ops_bwd = None
    from lv_xattn import ops
    real = ops.bwd
    try:
        ac._BWD_WS_CAP = ops.bwd_workspace_bytes(q, k, 300)      # forces chunks of 256 rows
        ops.bwd = lambda *a, **kw: (seen.append((a[10], a[11])), real(*a, **kw))[1]
        cut = lvx._attn_backward(do, q, k, v, o, L, False, w.scale, None, "flash", rounds=1, batched=True)
    finally:
        ops.bwd = real
        ac._BWD_WS_CAP = old
    torch.cuda.synchronize()
    assert seen == [(0, 256), (256, 256), (512, 256), (768, 256)]
    for g, g1, r, what in zip(cut, one, (ref["dq"], ref["dk"], ref["dv"]), ("dQ", "dK", "dV")):
        check_grad(g, r, what)
        assert (g.float() - g1.float()).abs().max() <= 2e-2 * r.abs().max()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("batched", [False, True])
def test_cfg0_shape_head_dim_64_runs_natively(lvx, batched, dtype, monkeypatch):
    """The CPU-only fp32 workload (head_dim 64, 4 rounds of 32 rows, 4096 keys) at its own
    shape, rounded to a 16-bit type: head_dim 64 has kernels of its own, so the operators get
    the tensors as they are (64 columns, nothing padded)."""
    from lv_xattn import ops
    dims = []
    real_fwd, real_bwd = ops.fwd, ops.bwd
    monkeypatch.setattr(ops, "fwd", lambda q_, *a, **kw: (dims.append(q_.shape[-1]), real_fwd(q_, *a, **kw))[1])
    monkeypatch.setattr(ops, "bwd", lambda q_, *a, **kw: (dims.append(q_.shape[-1]), real_bwd(q_, *a, **kw))[1])
    w = orc.make_inputs(orc.workload("cfg0"))
    assert w.D == 64 and abs(w.scale - 0.125) < 1e-12
    w.dtype = dtype
    w.tensors = {n: x.to(dtype) for n, x in w.tensors.items()}
    t = w.tensors
    ref = orc.layer_reference(w)
    q, k, v, do = (_dev(t[n]) for n in ("q", "k", "v", "do"))
    _, _, _, o, L = lvx._attn_forward(q, k, v, False, w.scale, None, rounds=w.rounds, batched=batched)
    dq, dk, dv = lvx._attn_backward(do, q, k, v, o, L, False, w.scale, None, "flash",
                                    rounds=w.rounds, batched=batched)
    torch.cuda.synchronize()
    assert dims and set(dims) == {64}
    assert o.shape == q.shape and o.is_contiguous() and o.dtype == dtype
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    check_o(o, ref["o"])
    check_lse(L, ref["lse"].reshape(w.B * w.Hq, w.Lq))
    check_grad(dq, ref["dq"], "dQ")
    check_grad(dk, ref["dk"], "dK")
    check_grad(dv, ref["dv"], "dV")


def test_head_dim_80_with_incoming_accumulator(lvx):
    """Head dimensions without kernels of their own pad to the next one that has (80 -> 128); the
    incoming accumulator pads with it."""
    g = torch.Generator().manual_seed(31)
    B, Hq, Hkv, D, Lq, Lkv = 2, 4, 2, 80, 96, 700
    q, k, v = (torch.randn(B, h, l, D, generator=g).bfloat16() for h, l in ((Hq, Lq), (Hkv, Lkv), (Hkv, Lkv)))
    k2, v2 = (torch.randn(B, Hkv, 300, D, generator=g).bfloat16() for _ in range(2))
    scale = D ** -0.5
    o_in, l_in = orc.attention_dense(q, k2, v2, scale)
    o_ref, l_ref = orc.attention_dense(q, torch.cat([k, k2], 2), torch.cat([v, v2], 2), scale)
    _, _, _, o, L = lvx._attn_forward(_dev(q), _dev(k), _dev(v), False, scale, None, rounds=3,
                                      acc_in=(_dev(o_in.bfloat16()), _dev(l_in.reshape(B * Hq, Lq))))
    torch.cuda.synchronize()
    assert o.shape == (B, Hq, Lq, D)
    check_o(o, o_ref)
    check_lse(L, l_ref.reshape(B * Hq, Lq))
    with pytest.raises(ValueError, match="exceeds 128"):
        lvx._attn_forward(_dev(torch.zeros(1, 2, 32, 160).bfloat16()), _dev(torch.zeros(1, 2, 64, 160).bfloat16()),
                          _dev(torch.zeros(1, 2, 64, 160).bfloat16()), False, 0.1, None, rounds=1)


@pytest.mark.parametrize("batched", [False, True])
def test_backward_masked_ragged_cfg4s(lvx, batched):
    w = orc.make_inputs(orc.workload("cfg4s"))
    t = w.tensors
    ref = orc.layer_reference(w)
    q, k, v, do = (_dev(t[n]) for n in ("q", "k", "v", "do"))
    mask = _mask_of(w, lvx)
    _, _, _, o, L = lvx._attn_forward(q, k, v, False, w.scale, None, rounds=w.rounds, mask=mask, batched=batched)
    dq, dk, dv = lvx._attn_backward(do, q, k, v, o, L, False, w.scale, None, "flash",
                                    rounds=w.rounds, mask=mask, batched=batched)
    torch.cuda.synchronize()
    check_grad(dq, ref["dq"], "dQ")
    check_grad(dk, ref["dk"], "dK")
    check_grad(dv, ref["dv"], "dV")
    dead = torch.isinf(ref["lse"])
    assert (dq.float().cpu()[dead] == 0).all()
    assert (dk.float().cpu()[1, :, w.kv_len[1]:] == 0).all() and (dv.float().cpu()[1, :, w.kv_len[1]:] == 0).all()


def test_backward_is_repeatable_up_to_atomic_order(lvx):
    w = orc.make_inputs(orc.workload("cfg1s"))
    t = w.tensors
    q, k, v, do = (_dev(t[n]) for n in ("q", "k", "v", "do"))
    _, _, _, o, L = lvx._attn_forward(q, k, v, False, w.scale, None, rounds=w.rounds)
    a = lvx._attn_backward(do, q, k, v, o, L, False, w.scale, None, "flash", rounds=w.rounds)
    b = lvx._attn_backward(do, q, k, v, o, L, False, w.scale, None, "flash", rounds=w.rounds)
    torch.cuda.synchronize()
    assert torch.equal(a[1], b[1]) and torch.equal(a[2], b[2])       # dK, dV: no atomics
    assert (a[0].float() - b[0].float()).abs().max() <= 2e-2 * a[0].float().abs().max()


# ------------------------------------------------------------------ recompute layer
@pytest.mark.parametrize("name", ["cfg2s", "cfg3s", "cfg2s_d64"])
def test_recompute_layer_autograd(lvx, name):
    w = orc.make_inputs(orc.workload(name))
    t = w.tensors
    ref = orc.layer_reference(w)
    attention = lvx.create_attention_class("lv_xattn", rounds=w.rounds, weight_grads=True).apply
    q = _dev(t["q"]).requires_grad_()
    x = _dev(t["x_vis"]).requires_grad_()
    wk = _dev(t["w_k"]).requires_grad_()
    wv = _dev(t["w_v"]).requires_grad_()
    o = attention(q, x, wk, wv, w.Hkv, w.scale)
    o.backward(_dev(t["do"]))
    torch.cuda.synchronize()
    check_o(o.detach(), ref["o"])
    check_grad(q.grad, ref["dq"], "dQ")
    check_grad(x.grad, ref["dx_vis"], "dX_vis")
    dwk_ref, dwv_ref = orc.dw_kv(t["x_vis"], ref["dk"].to(w.dtype), ref["dv"].to(w.dtype))
    check_grad(wk.grad, dwk_ref, "dW_k")
    check_grad(wv.grad, dwv_ref, "dW_v")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_recompute_layer_with_k_norm_autograd(lvx, dtype):
    w = orc.make_inputs(orc.workload("cfg2s"))
    w.dtype = dtype
    w.tensors = {n: (v.to(dtype) if v.is_floating_point() else v) for n, v in w.tensors.items()}
    t = w.tensors
    wn = (1.0 + 0.3 * torch.randn(w.D, generator=torch.Generator().manual_seed(9))).to(dtype)
    ref = orc.layer_reference(w, k_norm_weight=wn, k_norm_eps=1e-5)
    attention = lvx.create_attention_class("lv_xattn", rounds=w.rounds, weight_grads=True).apply
    q = _dev(t["q"]).requires_grad_()
    x = _dev(t["x_vis"]).requires_grad_()
    wk = _dev(t["w_k"]).requires_grad_()
    wv = _dev(t["w_v"]).requires_grad_()
    wnd = _dev(wn).requires_grad_()
    o = attention(q, x, wk, wv, w.Hkv, w.scale, None, wnd, 1e-5)
    o.backward(_dev(t["do"]))
    torch.cuda.synchronize()
    check_o(o.detach(), ref["o"])
    check_grad(q.grad, ref["dq"], "dQ")
    check_grad(x.grad, ref["dx_vis"], "dX_vis")
    check_grad(wnd.grad, ref["dw_norm"], "dw_norm")
    dwk_ref, dwv_ref = orc.dw_kv(t["x_vis"], ref["dk_raw"].to(w.dtype), ref["dv"].to(w.dtype))
    check_grad(wk.grad, dwk_ref, "dW_k")
    check_grad(wv.grad, dwv_ref, "dW_v")


def test_save_qkv_autograd_wrapper(lvx):
    w = orc.make_inputs(orc.workload("cfg1s"))
    t = w.tensors
    ref = orc.layer_reference(w)
    attention = lvx.create_attention_class_save_qkv("lv_xattn", rounds=w.rounds).apply
    q, k, v = (_dev(t[n]).requires_grad_() for n in ("q", "k", "v"))
    o = attention(q, k, v, False, w.scale)
    o.backward(_dev(t["do"]))
    torch.cuda.synchronize()
    check_o(o.detach(), ref["o"])
    check_grad(q.grad, ref["dq"], "dQ")
    check_grad(k.grad, ref["dk"], "dK")
    check_grad(v.grad, ref["dv"], "dV")


# ------------------------------------------------------------------ dense additive bias
@pytest.mark.parametrize("name", ["cfg2s", "cfg2s_d64"])
@pytest.mark.parametrize("batched", [False, True])
def test_dense_bias_forward_backward(lvx, batched, name):
    # the reference's bias_func path (lv_xattn/attn.py:386-389, 504-507): bias [B,1,Lq,Lkv]
    # added after the scale; here with a Llama-style -inf pattern plus finite noise, a row
    # that sees nothing, and a key length that is not a multiple of the tile; at head_dim 128 and 64
    w = orc.make_inputs(orc.workload(name))
    t = w.tensors
    B, Hq, Lq, Lkv = w.B, w.Hq, w.Lq, w.Lkv
    g = torch.Generator().manual_seed(77)
    bias = 0.5 * torch.randn(B, 1, Lq, Lkv, generator=g)
    bias[:, :, :, ::5] = float("-inf")
    bias[:, :, 7, :] = float("-inf")
    bias[:, :, 40:80, : Lkv // 2] = float("-inf")
    k, v = orc.kv_project(t["x_vis"], t["w_k"], t["w_v"], w.Hkv)
    k, v = k.to(w.dtype), v.to(w.dtype)
    o_ref, l_ref = orc.round_loop_forward(t["q"], k, v, w.scale, w.rounds, bias=bias)
    dq_ref, dk_ref, dv_ref = orc.attention_backward(t["do"], t["q"], k, v, o_ref, l_ref, w.scale, bias=bias,
                                                    rounds=w.rounds)
    calls = []

    def bias_func(local, remote):
        calls.append(1)
        return local + remote

    qd, kd, vd = _dev(t["q"]), _dev(k), _dev(v)
    la, ra = [_dev(bias)], [torch.zeros(1, device=DEV)]
    _, _, _, o, L = lvx._attn_forward(qd, kd, vd, False, w.scale, None, bias_func, la, ra, rounds=w.rounds,
                                      batched=batched)
    dq, dk, dv = lvx._attn_backward(_dev(t["do"]), qd, kd, vd, o, L, False, w.scale, None, "flash", bias_func, la, ra,
                                    rounds=w.rounds, batched=batched)
    torch.cuda.synchronize()
    assert len(calls) == 2
    check_o(o, o_ref)
    check_lse(L, l_ref)
    check_grad(dq, dq_ref, "dQ")
    check_grad(dk, dk_ref, "dK")
    check_grad(dv, dv_ref, "dV")
    dead = torch.isinf(l_ref)
    assert dead.any() and (o.float().cpu()[dead] == 0).all() and (dq.float().cpu()[dead] == 0).all()


@pytest.mark.parametrize("pure", [True, False])
def test_a_kept_bias_that_is_an_interval_mask_runs_without_the_bias(lvx, monkeypatch, pure):
    # what the Hugging Face hook hands over: the mask as a dense 0 / -inf bias that its maker keeps
    # for every layer (marked lvx_reused).  Tested once for being nothing but per-row intervals, it is
    # then dropped and the interval-mask kernels run; one finite entry inside a row's span keeps it.
    from lv_xattn import ops
    w = orc.make_inputs(orc.workload("cfg4s"))
    t = w.tensors
    allowed = orc.workload_allowed(w)                      # [B, Lq, Lkv] bool: an interval per row
    bias = torch.zeros(w.B, 1, w.Lq, w.Lkv).masked_fill_(~allowed.view(w.B, 1, w.Lq, w.Lkv), float("-inf"))
    if not pure:
        b0, r0 = allowed.any(-1).nonzero()[0].tolist()
        k0 = int(allowed[b0, r0].nonzero()[0])
        bias[b0, 0, r0, k0] = 0.25
    o_ref, l_ref = orc.round_loop_forward(t["q"], t["k"], t["v"], w.scale, w.rounds, bias=bias)
    dq_ref, dk_ref, dv_ref = orc.attention_backward(t["do"], t["q"], t["k"], t["v"], o_ref, l_ref, w.scale,
                                                    bias=bias, rounds=w.rounds)
    bias_d = _dev(bias)
    bias_d.lvx_reused = True
    seen = {"fwd": [], "bwd": [], "hull": 0}
    fwd0, bwd0, hull0 = ops.fwd, ops.bwd, ops.bias_hull
    monkeypatch.setattr(ops, "fwd", lambda *a, **kw: (seen["fwd"].append(a[11] if len(a) > 11 else kw.get("bias")), fwd0(*a, **kw))[1])
    monkeypatch.setattr(ops, "bwd", lambda *a, **kw: (seen["bwd"].append(kw.get("bias")), bwd0(*a, **kw))[1])
    monkeypatch.setattr(ops, "bias_hull", lambda *a, **kw: (seen.__setitem__("hull", seen["hull"] + 1), hull0(*a, **kw))[1])
    qd, kd, vd = _dev(t["q"]), _dev(t["k"]), _dev(t["v"])
    for _ in range(2):      # the second pass finds hull and verdict with the tensor
        _, _, _, o, L = lvx._attn_forward(qd, kd, vd, False, w.scale, None, lambda b: b, [bias_d], [], rounds=w.rounds)
        dq, dk, dv = lvx._attn_backward(_dev(t["do"]), qd, kd, vd, o, L, False, w.scale, None, "flash", lambda b: b,
                                        [bias_d], [], rounds=w.rounds)
    torch.cuda.synchronize()
    assert seen["hull"] == 1 and seen["fwd"] and seen["bwd"]
    assert all((b is None) == pure for b in seen["fwd"] + seen["bwd"])
    check_o(o, o_ref)
    check_lse(L, l_ref)
    check_grad(dq, dq_ref, "dQ")
    check_grad(dk, dk_ref, "dK")
    check_grad(dv, dv_ref, "dV")


@pytest.mark.gpu
@pytest.mark.parametrize("per_head,per_sample", [(False, True), (True, True), (False, False)])
def test_bias_hull_is_the_span_of_the_finite_entries(lvx, per_head, per_sample):
    """lvx_bias_hull against torch on a bias with -inf bands, an all -inf row, a row with one
    visible key and a key length that is not a multiple of 4; with it as the mask, forward and
    backward give what the dense-bias kernels give alone (the pairs outside the hull are exactly
    those a -inf bias removes)."""
    from lv_xattn import ops
    B, Hq, Hkv, Lq, Lkv, D = 2, 8, 2, 200, 1601, 128
    g = torch.Generator().manual_seed(5)
    bias = 0.3 * torch.randn(B if per_sample else 1, Hq if per_head else 1, Lq, Lkv, generator=g)
    for r in range(Lq):
        lo, hi = (r * 7) % 900, 901 + (r * 13) % 700
        bias[:, :, r, :lo] = float("-inf")
        bias[:, :, r, hi:] = float("-inf")
    if per_head:
        bias[:, 3, :, 100:300] = 0.25          # one head sees further to the left
    bias[:, :, 17, :] = float("-inf")
    bias[:, :, 18, :] = float("-inf")
    bias[:, :, 18, 1600] = 0.0
    bias[:, :, :, 400:500:3] = float("-inf")   # holes inside the hull stay the bias's business
    pad = torch.zeros(*bias.shape[:3], Lkv + 3)
    pad[..., :Lkv] = bias
    bias_d = pad.to(DEV)[..., :Lkv]
    q = (torch.randn(B, Hq, Lq, D, generator=g)).to(torch.bfloat16).to(DEV)
    k = (torch.randn(B, Hkv, Lkv, D, generator=g)).to(torch.bfloat16).to(DEV)
    v = (torch.randn(B, Hkv, Lkv, D, generator=g)).to(torch.bfloat16).to(DEV)
    do = (torch.randn(B, Hq, Lq, D, generator=g)).to(torch.bfloat16).to(DEV)
    m = ops.bias_hull(q, k, bias_d)
    live = ~torch.isinf(bias.expand(B, bias.shape[1], Lq, Lkv)).all(1) if per_head else ~torch.isinf(bias.expand(B, 1, Lq, Lkv))[:, 0]
    idx = torch.arange(Lkv).view(1, 1, -1)
    want_s = torch.where(live, idx, Lkv).amin(-1)
    want_e = torch.where(live, idx + 1, 0).amax(-1)
    want_s = torch.where(want_e > 0, want_s, 0)
    assert torch.equal(m.kv_start.cpu(), want_s.to(torch.int32)) and torch.equal(m.kv_end.cpu(), want_e.to(torch.int32))

    scale = D ** -0.5
    outs = []
    for mask in (None, m):
        o, L = torch.empty_like(q), torch.empty(B * Hq, Lq, device=DEV)
        ops.fwd(q, k, v, o, L, scale, mask=mask, bias=bias_d)
        delta = torch.empty_like(L)
        ops.bwd_preprocess(o, do, delta)
        dq = torch.empty_like(q)
        dk = torch.empty(B, Lkv, Hkv, D, dtype=torch.bfloat16, device=DEV).transpose(1, 2)
        dv = torch.empty_like(dk.transpose(1, 2)).transpose(1, 2)
        ws = torch.empty(ops.bwd_workspace_bytes(q, k, Lq, mask), dtype=torch.uint8, device=DEV)
        ops.bwd(q, k, v, do, L, delta, dq, dk, dv, scale, mask=mask, workspace=ws, bias=bias_d)
        outs.append((o, L, dq, dk, dv))
    torch.cuda.synchronize()
    (o0, L0, dq0, dk0, dv0), (o1, L1, dq1, dk1, dv1) = outs
    assert torch.equal(torch.isinf(L0), torch.isinf(L1)) and torch.isinf(L0).any()
    fin = ~torch.isinf(L0)
    assert (L0[fin] - L1[fin]).abs().max() <= 1e-5
    for a, b_, what in ((o0, o1, "O"), (dq0, dq1, "dQ"), (dk0, dk1, "dK"), (dv0, dv1, "dV")):
        ref = a.float().abs().max()
        assert (a.float() - b_.float()).abs().max() <= 4e-3 * ref, what
