"""CPU oracle for the per-GPU cross-attention hot path of LV-XAttn.

THIS IS TEST INFRASTRUCTURE.  Only the test-suite, the smoke check and the
``cpu_baseline`` leg of the benchmark may import it; the product path never
does and fails loudly when the HIP library is missing.

Every function restates, in plain fp32 PyTorch on the CPU, the arithmetic of a
piece of the reference (cited as ``file:line`` into the reference checkout).
The reference's kernels only run on a GPU under Triton, so nothing from it is
imported or executed; what pins this file is listed per function and exercised
by ``tests/test_oracle_*.py``:

* ``attention_dense``      - textbook softmax attention == the dense PyTorch
  check inside the reference's own harness (test.py:129-151).  Pinned against
  ``torch.nn.functional.scaled_dot_product_attention``, ``torch.logsumexp`` and
  a float64 brute-force loop.
* ``merge_lse``            - the rescale-merge of lv_xattn/attn.py:93-110 in
  max-subtracted form.  Pinned by identity / commutativity / associativity and
  by "split the keys, merge the parts == dense" on brute-force inputs.
* ``round_loop_forward``   - the P-round host loop of lv_xattn/attn.py:364-432
  with the ring exchange replaced by an index bump.
* ``attention_backward``   - the explicit formulas of
  lv_xattn/flash_attn_kernels.py:313-329 (delta) and :488-565 (P from LSE, dV,
  dP, dS, dK, dQ), accumulated per round as lv_xattn/attn.py:509-527 does.
  Pinned against ``torch.autograd`` through ``attention_dense`` and against
  central finite differences in float64.
* ``kv_project`` / ``dx_vis`` - the K/V projections of test_llama3.py:395-398
  (two GEMMs) and their input gradient (closed form; the reference drops this
  gradient, test_llama3.py:243).  Pinned against autograd.
* ``k_rms_norm`` / ``k_rms_norm_backward`` - the k_norm of test_llama3.py:418:
  MllamaTextRMSNorm of transformers 4.47.1 (requirements.txt:68; a dependency,
  absent from the reference checkout), whose published algorithm is
  w * (x * rsqrt(mean(x^2) + eps)) with the statistics in fp32.  Pinned against
  the MllamaTextRMSNorm class of the installed transformers, a hand-computed
  case, and (backward) autograd and float64 finite differences.

Reference quirks deliberately NOT restated (all are bugs or sit inside the
stated tolerance): the travelling LSE initialised to 0 instead of -inf
(attn.py:319), fp16 rounding of the scaled q and of P (attn.py:226,250), the
16-bit per-round rounding of O/dK/dV (attn.py:110,523-524), NaN on fully masked
rows (attn.py:245).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import torch

NEG_INF = float("-inf")


# --------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------
def expand_kv_heads(kv: torch.Tensor, n_q_heads: int) -> torch.Tensor:
    """[B,Hkv,L,D] -> [B,Hq,L,D]; q head h reads kv head h // (Hq/Hkv).

    Same head order as lv_xattn/attn.py:271-277 (expand on a new axis after the
    kv-head axis, then reshape)."""
    b, hkv, l, d = kv.shape
    if hkv == n_q_heads:
        return kv
    assert n_q_heads % hkv == 0
    return kv.repeat_interleave(n_q_heads // hkv, dim=1)


def reduce_kv_heads(dkv: torch.Tensor, n_kv_heads: int) -> torch.Tensor:
    """[B,Hq,L,D] -> [B,Hkv,L,D] by summing each group (attn.py:288-294)."""
    b, hq, l, d = dkv.shape
    if hq == n_kv_heads:
        return dkv
    return dkv.view(b, n_kv_heads, hq // n_kv_heads, l, d).sum(dim=2)


def interval_mask(kv_start: torch.Tensor, kv_end: torch.Tensor, lkv: int) -> torch.Tensor:
    """Boolean [B,Lq,Lkv]: True where text row i may attend visual token j,
    i.e. kv_start[b,i] <= j < kv_end[b,i]."""
    j = torch.arange(lkv).view(1, 1, lkv)
    return (j >= kv_start.unsqueeze(-1)) & (j < kv_end.unsqueeze(-1))


def _scores(q, k, scale, bias, allowed):
    s = torch.matmul(q.float(), k.float().transpose(-1, -2)) * scale  # attn.py:232-236: scale first
    if bias is not None:
        s = s + bias.float()                                            # attn.py:238-241: bias after scale
    if allowed is not None:
        s = s.masked_fill(~allowed.unsqueeze(1), NEG_INF)
    return s


# --------------------------------------------------------------------------
# forward
# --------------------------------------------------------------------------
def attention_dense(q, k, v, scale, bias=None, allowed=None):
    """Full-softmax attention of q [B,Hq,Lq,D] against k,v [B,Hkv,Lkv,D].

    Returns (O fp32 [B,Hq,Lq,D], LSE fp32 [B,Hq,Lq]) with
    LSE_i = ln sum_j exp(S_ij), O_i = sum_j exp(S_ij - LSE_i) V_j
    (natural-log LSE as attn.py:265-268).  Fully masked rows give O = 0 and
    LSE = -inf."""
    hq = q.shape[1]
    kf = expand_kv_heads(k, hq)
    vf = expand_kv_heads(v, hq)
    s = _scores(q, kf, scale, bias, allowed)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse.unsqueeze(-1))
    p = torch.nan_to_num(p, nan=0.0)          # rows with LSE = -inf
    o = torch.matmul(p, vf.float())
    return o, lse


def merge_lse(o_a, l_a, o_b, l_b):
    """Fold two partial results over disjoint key sets (attn.py:93-110):
    L' = ln(e^La + e^Lb),  O' = Oa e^(La-L') + Ob e^(Lb-L').

    Written with the maximum subtracted so that large LSE do not overflow and
    (-inf, -inf) stays (-inf, 0).  o_* [...,L,D], l_* [...,L]."""
    m = torch.maximum(l_a, l_b)
    m_safe = torch.where(torch.isinf(m) & (m < 0), torch.zeros_like(m), m)
    ea = torch.exp(l_a - m_safe)
    eb = torch.exp(l_b - m_safe)
    den = ea + eb
    l_new = m_safe + torch.log(den)
    l_new = torch.where(den == 0, torch.full_like(l_new, NEG_INF), l_new)
    wa = torch.where(den == 0, torch.zeros_like(den), ea / den)
    wb = torch.where(den == 0, torch.zeros_like(den), eb / den)
    o_new = o_a.float() * wa.unsqueeze(-1) + o_b.float() * wb.unsqueeze(-1)
    return o_new, l_new


def q_block_bounds(lq: int, rounds: int) -> List[Tuple[int, int]]:
    """Row windows of the P query blocks: ceil(Lq/P) rows each, the last ones
    shorter or empty (the reference requires Lq % P == 0, test.py:160)."""
    lb = -(-lq // rounds)
    return [(min(r * lb, lq), min((r + 1) * lb, lq)) for r in range(rounds)]


def round_loop_forward(q, k, v, scale, rounds, bias=None, allowed=None,
                       acc_in: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                       round_to_bf16: bool = False):
    """The P-round loop of attn.py:364-432 on one GPU's KV shard.

    Round r takes Q block r, computes its partial (O, LSE) against the whole
    local shard and folds it into the travelling accumulator of that block.
    ``acc_in`` is what would have arrived from the left neighbour; default is
    the identity (0, -inf).  Returns merged (O [B,Hq,Lq,D], LSE [B,Hq,Lq])."""
    b, hq, lq, d = q.shape
    o_out = torch.zeros(b, hq, lq, d)
    l_out = torch.full((b, hq, lq), NEG_INF)
    for (r0, r1) in q_block_bounds(lq, rounds):
        if r1 <= r0:
            continue
        bias_r = None if bias is None else bias[..., r0:r1, :]
        allowed_r = None if allowed is None else allowed[:, r0:r1]
        o_p, l_p = attention_dense(q[:, :, r0:r1], k, v, scale, bias_r, allowed_r)
        if round_to_bf16:
            o_p = o_p.bfloat16().float()
        if acc_in is None:
            o_a = torch.zeros_like(o_p)
            l_a = torch.full_like(l_p, NEG_INF)
        else:
            o_a, l_a = acc_in[0][:, :, r0:r1].float(), acc_in[1][:, :, r0:r1].float()
        o_m, l_m = merge_lse(o_a, l_a, o_p, l_p)
        o_out[:, :, r0:r1] = o_m
        l_out[:, :, r0:r1] = l_m
    return o_out, l_out


def split_kv_forward(q, k, v, scale, chunks: Sequence[Tuple[int, int]], bias=None, allowed=None):
    """Partial attention per key chunk folded sequentially with ``merge_lse``:
    what a ring of len(chunks) GPUs computes for one query block."""
    b, hq, lq, d = q.shape
    o_acc = torch.zeros(b, hq, lq, d)
    l_acc = torch.full((b, hq, lq), NEG_INF)
    for (c0, c1) in chunks:
        bias_c = None if bias is None else bias[..., c0:c1]
        allowed_c = None if allowed is None else allowed[:, :, c0:c1]
        o_p, l_p = attention_dense(q, k[:, :, c0:c1], v[:, :, c0:c1], scale, bias_c, allowed_c)
        o_acc, l_acc = merge_lse(o_acc, l_acc, o_p, l_p)
    return o_acc, l_acc


# --------------------------------------------------------------------------
# backward
# --------------------------------------------------------------------------
def bwd_delta(o, do):
    """delta_i = sum_d O_id dO_id (flash_attn_kernels.py:313-329)."""
    return (o.float() * do.float()).sum(dim=-1)


def attention_backward(do, q, k, v, o, lse, scale, bias=None, allowed=None, rounds: int = 1):
    """dQ, dK, dV from the saved, finally merged O and LSE.

    P_ij = exp(S_ij - LSE_i); dV_j = sum_i P_ij dO_i; dP_ij = dO_i . V_j;
    dS_ij = P_ij (dP_ij - delta_i); dQ_i = scale sum_j dS_ij K_j;
    dK_j = scale sum_i dS_ij Q_i  (flash_attn_kernels.py:488-565).
    The rows are visited in ``rounds`` blocks and dK/dV summed over them, as
    attn.py:509-527 does; dK/dV come back at Hkv heads (sum over the group)."""
    b, hq, lq, d = q.shape
    hkv = k.shape[1]
    kf = expand_kv_heads(k, hq).float()
    vf = expand_kv_heads(v, hq).float()
    dq = torch.zeros(b, hq, lq, d)
    dk = torch.zeros_like(kf)
    dv = torch.zeros_like(vf)
    delta = bwd_delta(o, do)
    for (r0, r1) in q_block_bounds(lq, rounds):
        if r1 <= r0:
            continue
        bias_r = None if bias is None else bias[..., r0:r1, :]
        allowed_r = None if allowed is None else allowed[:, r0:r1]
        qb = q[:, :, r0:r1].float()
        dob = do[:, :, r0:r1].float()
        s = _scores(qb, kf, scale, bias_r, allowed_r)
        p = torch.exp(s - lse[:, :, r0:r1].float().unsqueeze(-1))
        p = torch.nan_to_num(p, nan=0.0, posinf=0.0)
        dv += torch.matmul(p.transpose(-1, -2), dob)
        dp = torch.matmul(dob, vf.transpose(-1, -2))
        ds = p * (dp - delta[:, :, r0:r1].unsqueeze(-1))
        dq[:, :, r0:r1] = torch.matmul(ds, kf) * scale
        dk += torch.matmul(ds.transpose(-1, -2), qb) * scale
    return dq, reduce_kv_heads(dk, hkv), reduce_kv_heads(dv, hkv)


# --------------------------------------------------------------------------
# K/V recompute GEMMs
# --------------------------------------------------------------------------
def kv_project(x_vis, w_k, w_v, n_kv_heads: int):
    """K = X W_k, V = X W_v with X [B,Lkv,Dm], W [Dm, Hkv*D]; returned as
    [B,Hkv,Lkv,D] views (test_llama3.py:395-398 without the norms)."""
    b, l, dm = x_vis.shape
    k = torch.matmul(x_vis.float(), w_k.float())
    v = torch.matmul(x_vis.float(), w_v.float())
    d = k.shape[-1] // n_kv_heads
    return (k.view(b, l, n_kv_heads, d).transpose(1, 2),
            v.view(b, l, n_kv_heads, d).transpose(1, 2))


def dx_vis(dk, dv, w_k, w_v):
    """dX = dK W_k^T + dV W_v^T for dk, dv [B,Hkv,Lkv,D] (closed form; the
    reference returns no gradient here, test_llama3.py:243)."""
    b, hkv, l, d = dk.shape
    dk2 = dk.float().transpose(1, 2).reshape(b, l, hkv * d)
    dv2 = dv.float().transpose(1, 2).reshape(b, l, hkv * d)
    return torch.matmul(dk2, w_k.float().t()) + torch.matmul(dv2, w_v.float().t())


def dw_kv(x_vis, dk, dv):
    """dW_k = X^T dK, dW_v = X^T dV (summed over batch)."""
    b, hkv, l, d = dk.shape
    dk2 = dk.float().transpose(1, 2).reshape(b * l, hkv * d)
    dv2 = dv.float().transpose(1, 2).reshape(b * l, hkv * d)
    x2 = x_vis.float().reshape(b * l, -1)
    return torch.matmul(x2.t(), dk2), torch.matmul(x2.t(), dv2)


def k_rms_norm(k, weight, eps: float = 1e-5):
    """y = w * x * rsqrt(mean_d(x^2) + eps) over the last (head) dimension:
    `key_states = self.k_norm(key_states)`, test_llama3.py:418."""
    x = k.float()
    r = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return weight.float() * (x * r)


def k_rms_norm_backward(dy, k_raw, weight, eps: float = 1e-5):
    """(dx, dw) of k_rms_norm in closed form: with xh = x r and g = dy w,
    dx = r (g - xh mean_d(g xh)), dw = sum over all rows of dy xh."""
    x, dy, w = k_raw.float(), dy.float(), weight.float()
    r = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    xh = x * r
    g = dy * w
    dx = r * (g - xh * (g * xh).mean(-1, keepdim=True))
    dw = (dy * xh).reshape(-1, x.shape[-1]).sum(0)
    return dx, dw


# --------------------------------------------------------------------------
# workloads (the five configurations the build is measured and checked on)
# --------------------------------------------------------------------------
@dataclass
class Workload:
    name: str
    B: int
    Hq: int
    Hkv: int
    D: int
    Lq: int
    Lkv: int
    rounds: int
    dtype: torch.dtype = torch.bfloat16
    Dm: int = 0                      # > 0: K/V come from X_vis W
    sigma_x: float = 0.02
    q_len: Optional[List[int]] = None
    kv_len: Optional[List[int]] = None
    image_tokens: int = 0            # > 0: interval mask, tokens per image
    seed: int = 0
    tensors: dict = field(default_factory=dict)

    @property
    def scale(self) -> float:
        return 1.0 / math.sqrt(self.D)


def workload(name: str) -> Workload:
    """cfg0..cfg4 as the benchmark contract defines them, plus scaled-down
    siblings (suffix ``s``) the CPU oracle finishes in seconds."""
    table = {
        "cfg0": dict(B=1, Hq=8, Hkv=2, D=64, Lq=128, Lkv=4096, rounds=4, dtype=torch.float32),
        "cfg1": dict(B=1, Hq=32, Hkv=8, D=128, Lq=4096, Lkv=6404, rounds=16),
        "cfg2": dict(B=1, Hq=32, Hkv=8, D=128, Lq=4096, Lkv=6404, rounds=16, Dm=4096),
        "cfg3": dict(B=1, Hq=32, Hkv=8, D=128, Lq=2048, Lkv=65536, rounds=16, Dm=4096),
        "cfg4": dict(B=2, Hq=32, Hkv=8, D=128, Lq=3000, Lkv=6404, rounds=16,
                     q_len=[3000, 1777], kv_len=[6404, 3202], image_tokens=3202),
        # reduced siblings: same head structure and raggedness, fewer rows
        "cfg1s": dict(B=1, Hq=8, Hkv=2, D=128, Lq=512, Lkv=1601, rounds=4),
        "cfg2s": dict(B=1, Hq=8, Hkv=2, D=128, Lq=512, Lkv=1601, rounds=4, Dm=512),
        "cfg3s": dict(B=1, Hq=8, Hkv=2, D=128, Lq=256, Lkv=4096, rounds=16, Dm=512),
        "cfg2s_d64": dict(B=1, Hq=8, Hkv=2, D=64, Lq=512, Lkv=1601, rounds=4, Dm=512),   # cfg0's head_dim
        "cfg4s": dict(B=2, Hq=8, Hkv=2, D=128, Lq=375, Lkv=802, rounds=4,
                      q_len=[375, 222], kv_len=[802, 401], image_tokens=401),
    }
    return Workload(name=name, **table[name])


def make_inputs(w: Workload, need_grad_inputs: bool = True) -> Workload:
    """Seeded synthetic tensors, drawn on the CPU in fp32 in the fixed order
    Q, K, V, (X_vis, W_k, W_v), dO and then rounded to the workload dtype, so
    that the oracle and the GPU path see bit-identical inputs."""
    g = torch.Generator().manual_seed(w.seed)
    t = {}

    def draw(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(w.dtype)

    t["q"] = draw(w.B, w.Hq, w.Lq, w.D)
    k = draw(w.B, w.Hkv, w.Lkv, w.D)
    v = draw(w.B, w.Hkv, w.Lkv, w.D)
    if w.Dm > 0:
        t["x_vis"] = draw(w.B, w.Lkv, w.Dm, std=w.sigma_x)
        t["w_k"] = draw(w.Dm, w.Hkv * w.D, std=w.sigma_x)
        t["w_v"] = draw(w.Dm, w.Hkv * w.D, std=w.sigma_x)
    else:
        t["k"], t["v"] = k, v
    if need_grad_inputs:
        t["do"] = draw(w.B, w.Hq, w.Lq, w.D)
    if w.image_tokens > 0:
        t["kv_start"], t["kv_end"] = llama_intervals(w, g)
    w.tensors = t
    return w


def llama_intervals(w: Workload, g: torch.Generator):
    """Llama-3.2-style cross-attention mask in interval form: a text row
    attends only to the tokens of the most recent image placed before it; rows
    before the first image, and padding rows, attend to nothing.

    Image positions (the text row at which each image appears) are drawn from
    the seeded generator; image i of sample b occupies visual tokens
    [i*image_tokens, (i+1)*image_tokens)."""
    kv_start = torch.zeros(w.B, w.Lq, dtype=torch.int32)
    kv_end = torch.zeros(w.B, w.Lq, dtype=torch.int32)
    for b in range(w.B):
        ql = w.q_len[b] if w.q_len else w.Lq
        kl = w.kv_len[b] if w.kv_len else w.Lkv
        n_img = kl // w.image_tokens
        pos = torch.randint(1, max(ql - 1, 2), (n_img,), generator=g).sort().values.tolist()
        for i, p in enumerate(pos):
            nxt = pos[i + 1] if i + 1 < n_img else ql
            kv_start[b, p:nxt] = i * w.image_tokens
            kv_end[b, p:nxt] = (i + 1) * w.image_tokens
    return kv_start, kv_end


def workload_allowed(w: Workload) -> Optional[torch.Tensor]:
    """Boolean [B,Lq,Lkv] mask of a workload (None when everything is allowed)."""
    t = w.tensors
    if "kv_start" in t:
        return interval_mask(t["kv_start"].long(), t["kv_end"].long(), w.Lkv)
    if w.kv_len is not None:
        j = torch.arange(w.Lkv).view(1, 1, -1)
        return (j < torch.tensor(w.kv_len).view(-1, 1, 1)).expand(w.B, w.Lq, w.Lkv)
    return None


def n_pairs(w: Workload) -> int:
    """Unmasked (query row, key) pairs per q head, summed over the batch."""
    t = w.tensors
    if "kv_start" in t:
        return int((t["kv_end"].long() - t["kv_start"].long()).clamp(min=0).sum())
    if w.kv_len is not None:
        ql = w.q_len or [w.Lq] * w.B
        return int(sum(a * b for a, b in zip(ql, w.kv_len)))
    return w.B * w.Lq * w.Lkv


def layer_reference(w: Workload, backward: bool = True, rounds_bwd: Optional[int] = None,
                    k_norm_weight=None, k_norm_eps: float = 1e-5):
    """One cross-attention layer on the oracle: (K/V projection (+ k_norm),)
    round-loop forward, and optionally backward incl. dX_vis.  Returns a dict
    of fp32 tensors.  K/V are rounded to the workload dtype after the
    projection, as the device path stores them."""
    t = w.tensors
    out = {}
    k_raw = None
    if w.Dm > 0:
        k, v = kv_project(t["x_vis"], t["w_k"], t["w_v"], w.Hkv)
        k, v = k.to(w.dtype), v.to(w.dtype)
        if k_norm_weight is not None:
            k_raw = k
            k = k_rms_norm(k_raw, k_norm_weight, k_norm_eps).to(w.dtype)
        out["k"], out["v"] = k.float(), v.float()
    else:
        k, v = t["k"], t["v"]
    allowed = workload_allowed(w)
    o, lse = round_loop_forward(t["q"], k, v, w.scale, w.rounds, allowed=allowed)
    out["o"], out["lse"] = o, lse
    if backward:
        o_saved = o.to(w.dtype)
        dq, dk, dv = attention_backward(t["do"], t["q"], k, v, o_saved, lse, w.scale,
                                        allowed=allowed, rounds=rounds_bwd or w.rounds)
        out["dq"], out["dk"], out["dv"] = dq, dk, dv
        if w.Dm > 0:
            if k_raw is not None:
                dk, out["dw_norm"] = k_rms_norm_backward(dk.to(w.dtype), k_raw, k_norm_weight, k_norm_eps)
                out["dk_raw"] = dk
            out["dx_vis"] = dx_vis(dk.to(w.dtype), dv.to(w.dtype), t["w_k"], t["w_v"])
    return out
