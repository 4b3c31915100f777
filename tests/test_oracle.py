"""Pins the CPU oracle against things it does not itself define: library
routines, float64 brute force written from the definitions, autograd, finite
differences and algebraic invariants.  A dropped term, a wrong sign, a
transposed operand or a misplaced scale in the oracle fails one of these."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import lvx_oracle as orc


def _rand(*shape, seed=0, std=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def brute_force_attention(q, k, v, scale, bias=None, allowed=None):
    """Definition of softmax attention in float64 with explicit loops over
    (batch, head, row); written from the textbook formula, not from the
    oracle's code."""
    q, k, v = (t.double().numpy() for t in (q, k, v))
    B, Hq, Lq, D = q.shape
    Hkv, Lkv = k.shape[1], k.shape[2]
    G = Hq // Hkv
    O = np.zeros((B, Hq, Lq, D))
    L = np.full((B, Hq, Lq), -np.inf)
    for b in range(B):
        for h in range(Hq):
            for i in range(Lq):
                s = k[b, h // G] @ q[b, h, i] * scale
                if bias is not None:
                    bb = bias.double().numpy()
                    s = s + bb[b if bb.shape[0] > 1 else 0, h if bb.shape[1] > 1 else 0, i]
                if allowed is not None:
                    keep = allowed[b, i].numpy()
                    if not keep.any():
                        continue
                    s = np.where(keep, s, -np.inf)
                m = s.max()
                e = np.exp(s - m)
                L[b, h, i] = m + math.log(e.sum())
                O[b, h, i] = (e / e.sum()) @ v[b, h // G]
    return torch.from_numpy(O), torch.from_numpy(L)


# ---------------------------------------------------------------- forward
def test_dense_matches_sdpa_and_logsumexp():
    q, k, v = _rand(2, 4, 33, 64, seed=1), _rand(2, 4, 70, 64, seed=2), _rand(2, 4, 70, 64, seed=3)
    scale = 0.37
    o, lse = orc.attention_dense(q, k, v, scale)
    ref = F.scaled_dot_product_attention(q, k, v, scale=scale)
    assert torch.allclose(o, ref, atol=2e-6)
    assert torch.allclose(lse, torch.logsumexp(q @ k.transpose(-1, -2) * scale, -1), atol=2e-6)


def test_dense_gqa_bias_against_brute_force():
    # the reference harness' own case in miniature (test.py:101-107,273-288):
    # N(0,0.5) inputs, scale 0.5, additive bias with columns alternating 0/1
    q = _rand(1, 4, 9, 16, seed=4, std=0.5)
    k = _rand(1, 2, 21, 16, seed=5, std=0.5)
    v = _rand(1, 2, 21, 16, seed=6, std=0.5)
    bias = torch.zeros(1, 1, 9, 21)
    bias[..., 1::2] = 1.0
    o, lse = orc.attention_dense(q, k, v, 0.5, bias=bias)
    o_bf, l_bf = brute_force_attention(q, k, v, 0.5, bias=bias)
    assert torch.allclose(o.double(), o_bf, atol=1e-6)
    assert torch.allclose(lse.double(), l_bf, atol=1e-6)
    # head mapping: q heads 0,1 -> kv head 0; 2,3 -> kv head 1
    o2, _ = orc.attention_dense(q[:, 2:3], k[:, 1:2], v[:, 1:2], 0.5, bias=bias)
    assert torch.allclose(o[:, 2:3], o2, atol=1e-6)


def test_dense_masked_rows_zero_and_neg_inf():
    q, k, v = _rand(2, 2, 12, 8, seed=7), _rand(2, 1, 20, 8, seed=8), _rand(2, 1, 20, 8, seed=9)
    ks = torch.tensor([[0] * 4 + [5] * 8, [3] * 12])
    ke = torch.tensor([[0] * 4 + [11] * 8, [3] * 6 + [20] * 6])
    allowed = orc.interval_mask(ks, ke, 20)
    o, lse = orc.attention_dense(q, k, v, 0.3, allowed=allowed)
    o_bf, l_bf = brute_force_attention(q, k, v, 0.3, allowed=allowed)
    assert torch.isfinite(o).all()
    assert torch.allclose(o.double(), o_bf, atol=1e-6)
    assert torch.equal(torch.isinf(lse), torch.isinf(l_bf))
    fin = torch.isfinite(l_bf)
    assert torch.allclose(lse.double()[fin], l_bf[fin], atol=1e-6)
    assert (o[0, :, :4] == 0).all() and (lse[0, :, :4] == float("-inf")).all()


# ---------------------------------------------------------------- merge
def test_merge_identity_commutative_associative():
    o1, o2, o3 = (_rand(2, 3, 5, 8, seed=s) for s in (10, 11, 12))
    l1, l2, l3 = (_rand(2, 3, 5, seed=s, std=3.0) for s in (13, 14, 15))
    ident_o, ident_l = torch.zeros_like(o1), torch.full_like(l1, float("-inf"))
    o, l = orc.merge_lse(ident_o, ident_l, o1, l1)
    assert torch.equal(o, o1) and torch.equal(l, l1)
    o, l = orc.merge_lse(ident_o, ident_l, ident_o, ident_l)
    assert (o == 0).all() and (l == float("-inf")).all()
    oa, la = orc.merge_lse(o1, l1, o2, l2)
    ob, lb = orc.merge_lse(o2, l2, o1, l1)
    assert torch.allclose(oa, ob, atol=1e-6) and torch.allclose(la, lb, atol=1e-6)
    o12_3 = orc.merge_lse(*orc.merge_lse(o1, l1, o2, l2), o3, l3)
    o1_23 = orc.merge_lse(o1, l1, *orc.merge_lse(o2, l2, o3, l3))
    assert torch.allclose(o12_3[0], o1_23[0], atol=1e-5)
    assert torch.allclose(o12_3[1], o1_23[1], atol=1e-5)


def test_merge_matches_reference_formula_where_it_does_not_overflow():
    # literal form of attn.py:99,106 evaluated in float64
    o1, o2 = _rand(1, 2, 6, 4, seed=20), _rand(1, 2, 6, 4, seed=21)
    l1, l2 = _rand(1, 2, 6, seed=22, std=2.0), _rand(1, 2, 6, seed=23, std=2.0)
    ln = torch.log(torch.exp(l1.double()) + torch.exp(l2.double()))
    on = (o1.double() * torch.exp(l1.double())[..., None] / torch.exp(ln)[..., None]
          + o2.double() * torch.exp(l2.double())[..., None] / torch.exp(ln)[..., None])
    o, l = orc.merge_lse(o1, l1, o2, l2)
    assert torch.allclose(o.double(), on, atol=1e-6) and torch.allclose(l.double(), ln, atol=1e-6)
    # and it survives LSE values where the literal form overflows
    o, l = orc.merge_lse(o1, l1 + 200.0, o2, l2 + 200.0)
    assert torch.isfinite(o).all() and torch.allclose(l.double(), ln + 200.0, atol=1e-4)


def test_split_keys_then_merge_equals_dense():
    q, k, v = _rand(1, 4, 10, 16, seed=30), _rand(1, 2, 37, 16, seed=31), _rand(1, 2, 37, 16, seed=32)
    o_bf, l_bf = brute_force_attention(q, k, v, 0.25)
    o, l = orc.split_kv_forward(q, k, v, 0.25, [(0, 5), (5, 6), (6, 30), (30, 37)])
    assert torch.allclose(o.double(), o_bf, atol=1e-6) and torch.allclose(l.double(), l_bf, atol=1e-6)


def test_round_loop_cfg0_equals_full_softmax():
    # configuration 0: fp32, B1 Hq8 Hkv2 D64, Lq 128 = 4 x 32, Lkv 4096, seed 0
    w = orc.make_inputs(orc.workload("cfg0"))
    t = w.tensors
    o, l = orc.round_loop_forward(t["q"], t["k"], t["v"], w.scale, w.rounds)
    ref = F.scaled_dot_product_attention(t["q"], orc.expand_kv_heads(t["k"], 8),
                                         orc.expand_kv_heads(t["v"], 8), scale=w.scale)
    assert (o - ref).abs().max() < 1e-6
    s = torch.matmul(t["q"].double(), orc.expand_kv_heads(t["k"], 8).double().transpose(-1, -2)) * w.scale
    assert (l.double() - torch.logsumexp(s, -1)).abs().max() < 1e-5
    # with an incoming accumulator the result is the closed-form merge
    g = torch.Generator().manual_seed(99)
    o_in = torch.randn(1, 8, 128, 64, generator=g)
    l_in = torch.randn(1, 8, 128, generator=g) * 0.1 + math.log(4096) + 0.5
    o2, l2 = orc.round_loop_forward(t["q"], t["k"], t["v"], w.scale, w.rounds, acc_in=(o_in, l_in))
    wa = torch.exp(l_in.double() - torch.logaddexp(l_in.double(), l.double()))
    expect = o_in.double() * wa[..., None] + o.double() * (1 - wa)[..., None]
    assert (o2.double() - expect).abs().max() < 1e-5
    assert (l2.double() - torch.logaddexp(l_in.double(), l.double())).abs().max() < 1e-5


def test_round_loop_ragged_block_bounds():
    assert orc.q_block_bounds(3000, 16)[0] == (0, 188)
    assert orc.q_block_bounds(3000, 16)[-1] == (2820, 3000)
    assert orc.q_block_bounds(10, 4) == [(0, 3), (3, 6), (6, 9), (9, 10)]
    q, k, v = _rand(1, 2, 10, 8, seed=40), _rand(1, 2, 13, 8, seed=41), _rand(1, 2, 13, 8, seed=42)
    o, l = orc.round_loop_forward(q, k, v, 0.5, 4)
    o_d, l_d = orc.attention_dense(q, k, v, 0.5)
    assert torch.allclose(o, o_d, atol=1e-6) and torch.allclose(l, l_d, atol=1e-6)


# ---------------------------------------------------------------- backward
def _autograd_grads(q, k, v, do, scale, bias=None, allowed=None):
    q, k, v = (t.double().clone().requires_grad_() for t in (q, k, v))
    G = q.shape[1] // k.shape[1]
    kf, vf = k.repeat_interleave(G, 1), v.repeat_interleave(G, 1)
    s = q @ kf.transpose(-1, -2) * scale
    if bias is not None:
        s = s + bias.double()
    if allowed is not None:
        s = s.masked_fill(~allowed.unsqueeze(1), float("-inf"))
    p = torch.nan_to_num(torch.softmax(s, -1), nan=0.0)
    (p @ vf).backward(do.double())
    return q.grad, k.grad, v.grad


@pytest.mark.parametrize("rounds", [1, 3])
def test_backward_matches_autograd(rounds):
    q, k, v = _rand(2, 4, 9, 16, seed=50), _rand(2, 2, 14, 16, seed=51), _rand(2, 2, 14, 16, seed=52)
    do = _rand(2, 4, 9, 16, seed=53)
    bias = _rand(2, 1, 9, 14, seed=54)
    o, lse = orc.attention_dense(q, k, v, 0.4, bias=bias)
    dq, dk, dv = orc.attention_backward(do, q, k, v, o, lse, 0.4, bias=bias, rounds=rounds)
    gq, gk, gv = _autograd_grads(q, k, v, do, 0.4, bias=bias)
    assert torch.allclose(dq.double(), gq, atol=1e-5)
    assert torch.allclose(dk.double(), gk, atol=1e-5)
    assert torch.allclose(dv.double(), gv, atol=1e-5)


def test_backward_masked_rows_have_zero_grad():
    q, k, v = _rand(1, 2, 8, 8, seed=60), _rand(1, 1, 12, 8, seed=61), _rand(1, 1, 12, 8, seed=62)
    do = _rand(1, 2, 8, 8, seed=63)
    ks = torch.tensor([[0, 0, 0, 2, 2, 2, 6, 6]])
    ke = torch.tensor([[0, 0, 0, 6, 6, 6, 12, 12]])
    allowed = orc.interval_mask(ks, ke, 12)
    o, lse = orc.attention_dense(q, k, v, 0.5, allowed=allowed)
    dq, dk, dv = orc.attention_backward(do, q, k, v, o, lse, 0.5, allowed=allowed, rounds=2)
    gq, gk, gv = _autograd_grads(q, k, v, do, 0.5, allowed=allowed)
    assert torch.isfinite(dq).all() and (dq[:, :, :3] == 0).all()
    assert torch.allclose(dq.double(), gq, atol=1e-5)
    assert torch.allclose(dk.double(), gk, atol=1e-5)
    assert torch.allclose(dv.double(), gv, atol=1e-5)
    assert (dk[:, :, :2] == 0).all() and (dv[:, :, :2] == 0).all()


def test_backward_finite_differences_float64():
    # central differences of f = sum(O * dO) in float64, independent of autograd
    q, k, v = _rand(1, 2, 3, 4, seed=70), _rand(1, 1, 5, 4, seed=71), _rand(1, 1, 5, 4, seed=72)
    do = _rand(1, 2, 3, 4, seed=73)
    scale = 0.6

    def f(q_, k_, v_):
        o, _ = brute_force_attention(q_, k_, v_, scale)
        return float((o * do.double()).sum())

    o, lse = orc.attention_dense(q, k, v, scale)
    dq, dk, dv = orc.attention_backward(do, q, k, v, o, lse, scale)
    eps = 1e-5
    for name, t, g in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        td = t.double()
        for idx in [(0, 0, 0, 0), (0, t.shape[1] - 1, t.shape[2] - 1, 3), (0, 0, 1, 2)]:
            tp, tm = td.clone(), td.clone()
            tp[idx] += eps
            tm[idx] -= eps
            args_p = {"q": q.double(), "k": k.double(), "v": v.double()}
            args_m = dict(args_p)
            args_p[name], args_m[name] = tp, tm
            fd = (f(args_p["q"], args_p["k"], args_p["v"]) - f(args_m["q"], args_m["k"], args_m["v"])) / (2 * eps)
            assert abs(fd - float(g[idx])) < 1e-4, (name, idx, fd, float(g[idx]))


def test_delta_is_rowsum_of_o_do():
    o, do = _rand(1, 2, 5, 8, seed=80), _rand(1, 2, 5, 8, seed=81)
    d = orc.bwd_delta(o, do)
    assert torch.allclose(d, torch.einsum("bhld,bhld->bhl", o, do), atol=1e-6)


# ---------------------------------------------------------------- projections
def test_kv_project_and_dx_vis_match_autograd():
    x = _rand(2, 7, 12, seed=90).double().requires_grad_()
    wk, wv = _rand(12, 8, seed=91).double().requires_grad_(), _rand(12, 8, seed=92).double().requires_grad_()
    k, v = orc.kv_project(x.detach().float(), wk.detach().float(), wv.detach().float(), 2)
    assert k.shape == (2, 2, 7, 4)
    k_ref = (x @ wk).view(2, 7, 2, 4).transpose(1, 2)
    v_ref = (x @ wv).view(2, 7, 2, 4).transpose(1, 2)
    assert torch.allclose(k.double(), k_ref.detach(), atol=1e-5)
    dk, dv = _rand(2, 2, 7, 4, seed=93), _rand(2, 2, 7, 4, seed=94)
    ((k_ref * dk.double()).sum() + (v_ref * dv.double()).sum()).backward()
    dx = orc.dx_vis(dk, dv, wk.detach().float(), wv.detach().float())
    assert torch.allclose(dx.double(), x.grad, atol=1e-5)
    dwk, dwv = orc.dw_kv(x.detach().float(), dk, dv)
    assert torch.allclose(dwk.double(), wk.grad, atol=1e-5)
    assert torch.allclose(dwv.double(), wv.grad, atol=1e-5)


# ---------------------------------------------------------------- workloads
def test_workload_generators_are_deterministic_and_shaped():
    w = orc.make_inputs(orc.workload("cfg4s"))
    w2 = orc.make_inputs(orc.workload("cfg4s"))
    for key in w.tensors:
        assert torch.equal(w.tensors[key], w2.tensors[key])
    ks, ke = w.tensors["kv_start"], w.tensors["kv_end"]
    assert ks.shape == (2, 375) and ks.dtype == torch.int32
    assert (ke[1, 222:] == 0).all()                      # padding rows attend nothing
    assert (ke[0] - ks[0]).max() == 401 and (ke[0, 0] - ks[0, 0]) == 0
    assert (ke[1] <= 401).all()
    assert orc.n_pairs(w) == int(orc.workload_allowed(w).sum())
    w1 = orc.make_inputs(orc.workload("cfg1s"))
    assert orc.n_pairs(w1) == 512 * 1601


def test_layer_reference_small_gradients_vs_autograd():
    w = orc.make_inputs(orc.workload("cfg4s"))
    t = w.tensors
    out = orc.layer_reference(w)
    allowed = orc.workload_allowed(w)
    gq, gk, gv = _autograd_grads(t["q"].float(), t["k"].float(), t["v"].float(), t["do"].float(),
                                 w.scale, allowed=allowed)
    # the oracle feeds the bf16-rounded O into delta, autograd does not: loose
    for a, b in ((out["dq"], gq), (out["dk"], gk), (out["dv"], gv)):
        rel = (a.double() - b).norm() / b.norm()
        assert rel < 5e-3


def test_backward_with_bias_against_autograd():
    # additive bias (with -inf entries) enters P = softmax(scale*S + bias) and gets no
    # gradient: compare the hand-written backward with autograd through the dense formula
    g = torch.Generator().manual_seed(5)
    q = torch.randn(1, 4, 10, 16, generator=g).double().requires_grad_()
    k = torch.randn(1, 2, 14, 16, generator=g).double().requires_grad_()
    v = torch.randn(1, 2, 14, 16, generator=g).double().requires_grad_()
    do = torch.randn(1, 4, 10, 16, generator=g).double()
    bias = torch.randn(1, 1, 10, 14, generator=g).double()
    bias[0, 0, :, 3] = float("-inf")
    bias[0, 0, 2, :7] = float("-inf")
    ke, ve = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    s = 0.3 * q @ ke.transpose(-1, -2) + bias
    o = torch.softmax(s, -1) @ ve
    o.backward(do)
    o_r, lse = orc.attention_dense(q.detach().float(), k.detach().float(), v.detach().float(), 0.3, bias=bias.float())
    dq, dk, dv = orc.attention_backward(do.float(), q.detach().float(), k.detach().float(), v.detach().float(),
                                        o_r, lse, 0.3, bias=bias.float(), rounds=2)
    assert (o_r.double() - o.detach()).abs().max() < 1e-5
    assert (dq.double() - q.grad).abs().max() < 1e-4
    assert (dk.double() - k.grad).abs().max() < 1e-4
    assert (dv.double() - v.grad).abs().max() < 1e-4


def test_k_rms_norm_against_library_class_and_hand_case():
    # hand case: x = (3, 4, 0, 0), eps = 0 -> rms = sqrt(25/4) = 2.5 -> xh = (1.2, 1.6, 0, 0)
    y = orc.k_rms_norm(torch.tensor([[3.0, 4.0, 0.0, 0.0]]), torch.tensor([1.0, 0.5, 2.0, 2.0]), eps=0.0)
    assert torch.allclose(y, torch.tensor([[1.2, 0.8, 0.0, 0.0]]), atol=1e-6)
    from transformers.models.mllama.modeling_mllama import MllamaTextRMSNorm
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 3, 17, 128, generator=g) * 1.7
    norm = MllamaTextRMSNorm(128, eps=1e-5)
    with torch.no_grad():
        norm.weight.copy_(torch.randn(128, generator=g))
        assert torch.allclose(orc.k_rms_norm(x, norm.weight, 1e-5), norm(x), atol=1e-5, rtol=1e-5)


def test_k_rms_norm_backward_against_autograd_and_finite_differences():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, 2, 5, 128, generator=g, dtype=torch.float64).requires_grad_()
    w = torch.randn(128, generator=g, dtype=torch.float64).requires_grad_()
    dy = torch.randn(2, 2, 5, 128, generator=g, dtype=torch.float64)
    y = w * x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5)
    y.backward(dy)
    dx, dw = orc.k_rms_norm_backward(dy, x.detach(), w.detach(), 1e-5)
    assert torch.allclose(dx.double(), x.grad, atol=1e-5, rtol=1e-4)
    assert torch.allclose(dw.double(), w.grad, atol=1e-4, rtol=1e-4)
    # one directional finite difference in float64 through the oracle's forward
    xd = x.detach()
    u = torch.randn_like(xd)
    h = 1e-3
    f = lambda t: (orc.k_rms_norm(t.float(), w.detach().float(), 1e-5).double() * dy).sum()
    fd = (f(xd + h * u) - f(xd - h * u)) / (2 * h)
    assert abs(fd - (x.grad * u).sum()) < 2e-2 * max(1.0, abs(fd))
