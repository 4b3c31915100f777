"""The generated check of the reference's own harness (test.py:101-107, 129-151,
192, 248-249, 273-288 there), restated for one GPU: fp16, H = 16 heads of 128,
L_Q = 1024, L_KV = 4096, q/k/v ~ N(0, 0.5^2), dO ~ N(0, 1), sm_scale = 0.5, the
additive bias that is 1 on every odd key column, compared with dense softmax
attention by torch.allclose(atol=1e-2, rtol=1e-3) - through the save-(q,k,v)
autograd wrapper with the reference's call signature, bias_func included.
Nothing of the reference is imported; its dense check is three lines of
PyTorch, which the oracle's `attention_dense` restates."""
import pytest
import torch

from oracle import lvx_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ATOL, RTOL = 1e-2, 1e-3          # test.py:248-249


def _bias_func(shape, val):       # test.py:276-279, evaluated on the device
    bias = torch.zeros([int(x) for x in shape], device=DEV)
    bias[:, :, :, 1::2] = val
    return bias


# the harness runs seeds 1..15 (test.py:101, 243); here with 4 query blocks, seed 1 also as one block
@pytest.mark.parametrize("seed,rounds", [(s, 4) for s in range(1, 16)] + [(1, 1)])
def test_reference_harness_check_fp16_with_bias(seed, rounds):
    import lv_xattn
    from lv_xattn import _lib
    _lib.load()
    Z, H, L_Q, L_KV, D = 1, 16, 1024, 4096, 128
    g = torch.Generator().manual_seed(seed)
    q = (0.5 * torch.randn(Z, H, L_Q, D, generator=g)).half()
    k = (0.5 * torch.randn(Z, H, L_KV, D, generator=g)).half()
    v = (0.5 * torch.randn(Z, H, L_KV, D, generator=g)).half()
    dout = torch.randn(Z, H, L_Q, D, generator=g).half()
    sm_scale = 0.5
    ref_bias = torch.zeros(L_Q, L_KV)
    ref_bias[:, 1::2] = 1

    o_ref, lse_ref = orc.attention_dense(q, k, v, sm_scale, bias=ref_bias[None, None])
    dq_ref, dk_ref, dv_ref = orc.attention_backward(dout, q, k, v, o_ref.half(), lse_ref, sm_scale,
                                                    bias=ref_bias[None, None])

    attention = lv_xattn.create_attention_class_save_qkv("lv_xattn", rounds=rounds).apply
    qd, kd, vd = (t.to(DEV).requires_grad_() for t in (q, k, v))
    # the shape argument covers all rows held here (the reference passes one rank's block)
    local_bias_args = [torch.tensor([Z, 1, L_Q, L_KV])]
    remote_bias_args = [torch.tensor(1)]
    out = attention(qd, kd, vd, False, sm_scale, _bias_func, local_bias_args, remote_bias_args).half()
    assert torch.allclose(out.float().cpu(), o_ref, atol=ATOL, rtol=RTOL)
    out.backward(dout.to(DEV))
    torch.cuda.synchronize()
    for name, got, ref in (("dq", qd.grad, dq_ref), ("dk", kd.grad, dk_ref), ("dv", vd.grad, dv_ref)):
        assert torch.allclose(got.float().cpu(), ref, atol=ATOL, rtol=RTOL), \
            f"{name}: max-abs {(got.float().cpu() - ref).abs().max().item():.3e}"
