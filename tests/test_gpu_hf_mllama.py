"""The Hugging Face Mllama cross-attention layer with the "lv_xattn" attention
implementation against the same layer with transformers' own eager attention
(an implementation independent of this repository's oracle): forward output
and every parameter / input gradient."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _layer(impl, dtype=torch.bfloat16):
    from transformers.models.mllama import modeling_mllama as m
    from transformers.models.mllama.configuration_mllama import MllamaTextConfig
    cfg = MllamaTextConfig(hidden_size=1024, num_attention_heads=8, num_key_value_heads=2, num_hidden_layers=2,
                           intermediate_size=256, cross_attention_layers=[1], vocab_size=128,
                           bos_token_id=1, eos_token_id=2, pad_token_id=0)
    cfg._attn_implementation = impl
    torch.manual_seed(3)
    layer = m.MllamaTextCrossAttention(cfg, layer_idx=1)
    with torch.no_grad():          # norm weights other than the all-ones initialisation
        layer.q_norm.weight.copy_(1.0 + 0.3 * torch.randn(128))
        layer.k_norm.weight.copy_(1.0 + 0.3 * torch.randn(128))
    return layer.to(device=DEV, dtype=dtype)


@pytest.mark.parametrize("variant,dtype", [("interface", torch.bfloat16), ("recompute", torch.bfloat16),
                                           ("recompute_intervals", torch.bfloat16),
                                           ("interface", torch.float16), ("recompute", torch.float16)])
def test_mllama_cross_attention_layer_matches_eager(variant, dtype):
    """interface: the attention-interface hook (K/V kept for backward);
    recompute: the patched forward (K/V + k_norm recomputed by the fused GEMM),
    with the dense mask or with the same mask as per-row key intervals."""
    pytest.importorskip("transformers")
    import lv_xattn
    from lv_xattn import _lib, hf_mllama
    _lib.load()
    name = hf_mllama.register()
    ref, new = _layer("eager", dtype), _layer(name, dtype)
    new.load_state_dict(ref.state_dict())
    assert ref.head_dim == 128
    if variant != "interface":
        assert hf_mllama.patch_cross_attention_forward(new) == 1

    g = torch.Generator().manual_seed(11)
    B, Lq, Lkv = 2, 200, 1601
    x = torch.randn(B, Lq, 1024, generator=g).to(dtype).to(DEV)
    vis = torch.randn(B, Lkv, 1024, generator=g).to(dtype).to(DEV)
    go = torch.randn(B, Lq, 1024, generator=g).to(dtype).to(DEV)
    # Llama-3.2 style additive mask: rows before the image see nothing (all entries
    # at the dtype minimum, as transformers builds it), sample 1 sees only the first tile
    neg = torch.finfo(dtype).min
    mask = torch.zeros(B, 1, Lq, Lkv, dtype=dtype)
    mask[0, :, :17, :] = neg
    mask[1, :, :, 800:] = neg
    mask = mask.to(DEV)
    # rows masked everywhere are zeroed by the decoder layer right after the attention
    # (full_text_row_masked_out_mask); what they hold before that is implementation-defined
    # (uniform attention in eager, score-weighted here and in the reference), so they get
    # no output gradient and are left out of the output comparison
    live = (mask[:, 0] > neg / 2).any(-1)                  # [B, Lq]
    go = go * live[..., None]

    extra = {}
    if variant == "recompute_intervals":
        start = torch.zeros(B, Lq, dtype=torch.int32)
        end = torch.full((B, Lq), Lkv, dtype=torch.int32)
        end[0, :17] = 0
        end[1, :] = 800
        extra["lvx_mask"] = lv_xattn.Mask(None, start.to(DEV), end.to(DEV))

    outs = []
    for layer in (ref, new):
        xi, vi = x.clone().requires_grad_(), vis.clone().requires_grad_()
        o, _ = layer(xi, cross_attention_states=vi, attention_mask=mask, **(extra if layer is new else {}))
        o.backward(go)
        torch.cuda.synchronize()
        outs.append((o.detach().float(), xi.grad.float(), vi.grad.float(),
                     {n: p.grad.float() for n, p in layer.named_parameters()}))
        layer.zero_grad()
    (o_r, dx_r, dv_r, gp_r), (o_n, dx_n, dv_n, gp_n) = outs

    def rel(a, b):
        return ((a - b).norm() / b.norm().clamp_min(1e-12)).item()

    # both sides are bf16 pipelines; the eager one rounds P to bf16 before P V as well
    lv = live[..., None].float()
    assert rel(o_n * lv, o_r * lv) < 2e-2
    assert rel(dx_n, dx_r) < 3e-2
    assert rel(dv_n, dv_r) < 3e-2
    for n in gp_r:
        assert rel(gp_n[n], gp_r[n]) < 3e-2, n
