"""The Hugging Face Mllama cross-attention layer with the "lv_xattn" attention
implementation against the same layer with transformers' own eager attention
(an implementation independent of this repository's oracle): forward output
and every parameter / input gradient."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _layer(impl, dtype=torch.bfloat16, hidden=1024):
    from transformers.models.mllama import modeling_mllama as m
    from transformers.models.mllama.configuration_mllama import MllamaTextConfig
    cfg = MllamaTextConfig(hidden_size=hidden, num_attention_heads=8, num_key_value_heads=2, num_hidden_layers=2,
                           intermediate_size=256, cross_attention_layers=[1], vocab_size=128,
                           bos_token_id=1, eos_token_id=2, pad_token_id=0)
    cfg._attn_implementation = impl
    torch.manual_seed(3)
    layer = m.MllamaTextCrossAttention(cfg, layer_idx=1)
    with torch.no_grad():          # norm weights other than the all-ones initialisation
        layer.q_norm.weight.copy_(1.0 + 0.3 * torch.randn(hidden // 8))
        layer.k_norm.weight.copy_(1.0 + 0.3 * torch.randn(hidden // 8))
    return layer.to(device=DEV, dtype=dtype)


@pytest.mark.parametrize("variant,dtype,hidden", [("interface", torch.bfloat16, 1024), ("recompute", torch.bfloat16, 1024),
                                                  ("recompute_intervals", torch.bfloat16, 1024),
                                                  ("interface", torch.float16, 1024), ("recompute", torch.float16, 1024),
                                                  ("interface", torch.bfloat16, 512)])
def test_mllama_cross_attention_layer_matches_eager(variant, dtype, hidden):
    """interface: the attention-interface hook (K/V kept for backward), also with heads of 64
    (hidden size 512);
    recompute: the patched forward (K/V + k_norm recomputed by the fused GEMM),
    with the dense mask or with the same mask as per-row key intervals."""
    pytest.importorskip("transformers")
    import lv_xattn
    from lv_xattn import _lib, hf_mllama
    _lib.load()
    name = hf_mllama.register()
    ref, new = _layer("eager", dtype, hidden), _layer(name, dtype, hidden)
    new.load_state_dict(ref.state_dict())
    assert ref.head_dim == hidden // 8
    if variant != "interface":
        assert hf_mllama.patch_cross_attention_forward(new) == 1

    g = torch.Generator().manual_seed(11)
    B, Lq, Lkv = 2, 200, 1601
    x = torch.randn(B, Lq, hidden, generator=g).to(dtype).to(DEV)
    vis = torch.randn(B, Lkv, hidden, generator=g).to(dtype).to(DEV)
    go = torch.randn(B, Lq, hidden, generator=g).to(dtype).to(DEV)
    # Llama-3.2 style additive mask: rows before the image see nothing (all entries
    # at the dtype minimum, as transformers builds it), sample 1 sees only the first tile
    neg = torch.finfo(dtype).min
    mask = torch.zeros(B, 1, Lq, Lkv, dtype=dtype)
    mask[0, :, :17, :] = neg
    mask[1, :, :, 800:] = neg
    mask = mask.to(DEV)
    # rows masked everywhere do not occur in the masks transformers prepares (it turns them
    # into rows that see everything); what an implementation returns for them is its own
    # business (uniform attention in eager, score-weighted here and in the reference), so
    # they get no output gradient and are left out of the output comparison
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


@pytest.mark.parametrize("variant", ["interface", "recompute", "recompute_intervals"])
def test_tiny_mllama_text_model_matches_eager(variant):
    """A four-layer MllamaForCausalLM (two self-attention, two cross-attention decoder layers,
    random weights) end to end.  Truth is the model in fp32 with transformers' eager attention;
    the bf16 model with the "lv_xattn" implementation (interface hook, or the patched recompute
    forward on both cross-attention layers, there also with the mask handed through the model's
    keyword arguments as per-row key intervals) must come as close to it as the bf16 model with
    eager attention does (within a factor 2), in the logits and in every gradient."""
    pytest.importorskip("transformers")
    from transformers.models.mllama import modeling_mllama as m
    from transformers.models.mllama.configuration_mllama import MllamaTextConfig
    from lv_xattn import _lib, hf_mllama
    _lib.load()
    name = hf_mllama.register()

    def build(impl, dtype):
        cfg = MllamaTextConfig(hidden_size=1024, num_attention_heads=8, num_key_value_heads=2, num_hidden_layers=4,
                               intermediate_size=256, cross_attention_layers=[1, 3], vocab_size=128,
                               bos_token_id=1, eos_token_id=2, pad_token_id=0, max_position_embeddings=512)
        cfg._attn_implementation = impl
        torch.manual_seed(5)
        model = m.MllamaForCausalLM(cfg)
        with torch.no_grad():      # the gates start at zero, which would switch cross-attention off
            for layer in model.model.layers:
                if hasattr(layer, "cross_attn_attn_gate"):
                    layer.cross_attn_attn_gate.fill_(0.7)
                    layer.cross_attn_mlp_gate.fill_(0.4)
        return model.to(device=DEV, dtype=dtype)

    truth, ref, new = build("eager", torch.float32), build("eager", torch.bfloat16), build(name, torch.bfloat16)
    ref.load_state_dict(truth.state_dict())          # the same bf16-rounded weights in both bf16 models
    new.load_state_dict(ref.state_dict())
    truth.load_state_dict(ref.state_dict())          # and those exact values in the fp32 one
    if variant != "interface":
        assert hf_mllama.patch_cross_attention_forward(new) == 2

    g = torch.Generator().manual_seed(21)
    B, Lq, Lkv = 2, 150, 1601
    ids = torch.randint(3, 128, (B, Lq), generator=g).to(DEV)
    vis = torch.randn(B, Lkv, 1024, generator=g).bfloat16().to(DEV)
    go = torch.randn(B, Lq, 128, generator=g).bfloat16().to(DEV)
    allowed = torch.ones(B, 1, Lq, Lkv, dtype=torch.bool)
    allowed[0, :, :9, :] = False               # text before the image
    allowed[1, :, :, 800:] = False             # one tile only
    allowed = allowed.to(DEV)

    res = []
    for model, dtype in ((truth, torch.float32), (ref, torch.bfloat16), (new, torch.bfloat16)):
        # as _prepare_cross_attention_mask builds them: rows that see no tile end up seeing all
        full = allowed.any(-1).to(dtype)[..., None]                   # [B, 1, Lq, 1]
        cmask = torch.zeros(B, 1, Lq, Lkv, dtype=dtype, device=DEV).masked_fill(~allowed, torch.finfo(dtype).min) * full
        v = vis.to(dtype).clone().requires_grad_()
        extra = {}
        if model is new and variant == "recompute_intervals":
            # the processor's form of the same mask: [B, T, images, tiles], one image of two tiles
            cam = torch.zeros(B, Lq, 1, 2, dtype=torch.int64)
            cam[0, 9:] = 1
            cam[1, :, 0, 0] = 1
            extra["lvx_mask"] = hf_mllama.mask_from_cross_attention_mask(cam.to(DEV), 800, kv_len=torch.tensor([Lkv, Lkv]))
            cmask = torch.zeros_like(cmask)      # the dense mask says nothing: only the intervals can get it right
        out = model(input_ids=ids, cross_attention_states=v, cross_attention_mask=cmask,
                    full_text_row_masked_out_mask=full, use_cache=False, **extra)
        (out.logits.float() * go.float()).sum().backward()
        torch.cuda.synchronize()
        grads = {n: p.grad.float() for n, p in model.named_parameters() if p.grad is not None}
        grads["cross_attention_states"] = v.grad.float()
        res.append((out.logits.detach().float(), grads))
        model.zero_grad()
    (lo_t, g_t), (lo_r, g_r), (lo_n, g_n) = res

    def rel(a, b):
        return ((a - b).norm() / b.norm().clamp_min(1e-12)).item()

    assert torch.isfinite(lo_n).all()
    assert rel(lo_r, lo_t) < 3e-2                   # the yardstick itself is sane
    assert rel(lo_n, lo_t) <= 2 * rel(lo_r, lo_t), (rel(lo_n, lo_t), rel(lo_r, lo_t))
    assert set(g_n) == set(g_t)
    bad = []
    for n in g_t:
        e_new, e_ref = rel(g_n[n], g_t[n]), rel(g_r[n], g_t[n])
        print(f"{n:60s} numel {g_t[n].numel():8d}  new {e_new:.4f}  eager-bf16 {e_ref:.4f}")
        # a gate is one number, the sum of a million products that largely cancel: its relative
        # error is the luck of the rounding (it moves between 2 % and 6 % with the order of the
        # fp32 sums inside the kernels, the eager bf16 model's own being 2.5 %), so it gets a wider floor
        floor = 1e-2 if g_t[n].numel() > 1 else 8e-2
        if e_new > max(2 * e_ref, floor):
            bad.append((n, e_new, e_ref))
    assert not bad, bad


@pytest.mark.parametrize("variant", ["interface", "recompute"])
def test_tiny_mllama_prefill_then_decode_with_cache(variant):
    """Inference with a K/V cache: a prefill over the prompt (cross-attention states given),
    then two single-token steps that read the cached cross-attention K/V (no states given).
    Logits of every step against the same bf16 model with eager attention."""
    pytest.importorskip("transformers")
    from transformers import DynamicCache
    from transformers.models.mllama import modeling_mllama as m
    from transformers.models.mllama.configuration_mllama import MllamaTextConfig
    from lv_xattn import _lib, hf_mllama
    _lib.load()
    name = hf_mllama.register()

    def build(impl):
        cfg = MllamaTextConfig(hidden_size=1024, num_attention_heads=8, num_key_value_heads=2, num_hidden_layers=4,
                               intermediate_size=256, cross_attention_layers=[1, 3], vocab_size=128,
                               bos_token_id=1, eos_token_id=2, pad_token_id=0, max_position_embeddings=512)
        cfg._attn_implementation = impl
        torch.manual_seed(9)
        model = m.MllamaForCausalLM(cfg)
        with torch.no_grad():
            for layer in model.model.layers:
                if hasattr(layer, "cross_attn_attn_gate"):
                    layer.cross_attn_attn_gate.fill_(0.7)
                    layer.cross_attn_mlp_gate.fill_(0.4)
        return model.to(device=DEV, dtype=torch.bfloat16).eval()

    ref, new = build("eager"), build(name)
    new.load_state_dict(ref.state_dict())
    if variant == "recompute":
        assert hf_mllama.patch_cross_attention_forward(new) == 2

    g = torch.Generator().manual_seed(33)
    B, Lq, Lkv, steps = 2, 70, 1601, 2
    ids = torch.randint(3, 128, (B, Lq + steps), generator=g).to(DEV)
    vis = torch.randn(B, Lkv, 1024, generator=g).bfloat16().to(DEV)
    allowed = torch.ones(B, 1, Lq + steps, Lkv, dtype=torch.bool)
    allowed[0, :, :5, :] = False
    allowed[1, :, :, 800:] = False
    full = allowed.any(-1).to(torch.bfloat16)[..., None].to(DEV)
    cmask = (torch.zeros(B, 1, Lq + steps, Lkv, dtype=torch.bfloat16)
             .masked_fill(~allowed, torch.finfo(torch.bfloat16).min).to(DEV)) * full

    def rel(a, b):
        return ((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-12)).item()

    outs = []
    with torch.no_grad():
        for model in (ref, new):
            cache = DynamicCache(config=model.config)
            lo = [model(input_ids=ids[:, :Lq], cross_attention_states=vis, cross_attention_mask=cmask[:, :, :Lq],
                        full_text_row_masked_out_mask=full[:, :, :Lq], past_key_values=cache, use_cache=True).logits]
            for t in range(Lq, Lq + steps):
                lo.append(model(input_ids=ids[:, t:t + 1], cross_attention_mask=cmask[:, :, t:t + 1],
                                full_text_row_masked_out_mask=full[:, :, t:t + 1], past_key_values=cache,
                                use_cache=True).logits)
            torch.cuda.synchronize()
            outs.append(lo)
    for step, (a, b) in enumerate(zip(outs[1], outs[0])):
        assert a.shape == b.shape and torch.isfinite(a).all()
        assert rel(a, b) < 3e-2, (step, rel(a, b))


def test_tiny_mllama_left_padded_batch():
    """A left-padded batch: the self-attention layers, which reach the hook under the same
    implementation name, must see transformers' causal + padding mask (a custom name gets none
    unless a mask builder is registered with it).  Logits at the real tokens against the eager
    model, with transformers' own SDPA model as the yardstick."""
    pytest.importorskip("transformers")
    from transformers.models.mllama import modeling_mllama as m
    from transformers.models.mllama.configuration_mllama import MllamaTextConfig
    from lv_xattn import _lib, hf_mllama
    _lib.load()
    name = hf_mllama.register()

    def build(impl):
        cfg = MllamaTextConfig(hidden_size=1024, num_attention_heads=8, num_key_value_heads=2, num_hidden_layers=4,
                               intermediate_size=256, cross_attention_layers=[1, 3], vocab_size=128,
                               bos_token_id=1, eos_token_id=2, pad_token_id=0, max_position_embeddings=512)
        cfg._attn_implementation = impl
        torch.manual_seed(5)
        model = m.MllamaForCausalLM(cfg)
        with torch.no_grad():
            for layer in model.model.layers:
                if hasattr(layer, "cross_attn_attn_gate"):
                    layer.cross_attn_attn_gate.fill_(0.7)
                    layer.cross_attn_mlp_gate.fill_(0.4)
        return model.to(device=DEV, dtype=torch.bfloat16).eval()

    ref, new, sdpa = build("eager"), build(name), build("sdpa")
    new.load_state_dict(ref.state_dict())
    sdpa.load_state_dict(ref.state_dict())
    g = torch.Generator().manual_seed(3)
    B, Lq, Lkv, pad = 2, 90, 1601, 25
    ids = torch.randint(3, 128, (B, Lq), generator=g)
    ids[1, :pad] = 0
    am = torch.ones(B, Lq, dtype=torch.long)
    am[1, :pad] = 0
    vis = torch.randn(B, Lkv, 1024, generator=g).bfloat16().to(DEV)
    allowed = torch.ones(B, 1, Lq, Lkv, dtype=torch.bool)
    allowed[0, :, :9] = False
    allowed[1, :, :, 800:] = False
    full = allowed.any(-1).to(torch.bfloat16)[..., None].to(DEV)
    cmask = torch.zeros(B, 1, Lq, Lkv, dtype=torch.bfloat16).masked_fill(~allowed, torch.finfo(torch.bfloat16).min).to(DEV) * full
    outs = []
    with torch.no_grad():
        for model in (ref, new, sdpa):
            outs.append(model(input_ids=ids.to(DEV), attention_mask=am.to(DEV), cross_attention_states=vis,
                              cross_attention_mask=cmask, full_text_row_masked_out_mask=full,
                              use_cache=False).logits.float())
    torch.cuda.synchronize()
    valid = am.bool().to(DEV)

    def rel(a, b):
        return ((a - b)[valid].norm() / b[valid].norm()).item()

    assert torch.isfinite(outs[1][valid]).all()
    assert rel(outs[1], outs[0]) <= max(2 * rel(outs[2], outs[0]), 1e-2), (rel(outs[1], outs[0]), rel(outs[2], outs[0]))
