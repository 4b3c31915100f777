"""Shared helpers of the GPU parity tests: tolerances and comparisons."""
import torch

# Tolerances of the build contract, vs the fp32 oracle on identical bf16 inputs.
O_MAX_ABS = 2e-2
O_MEAN_ABS = 2e-3
LSE_ABS = 1e-3
GRAD_REL_L2 = 1e-2


def check_o(o_dev: torch.Tensor, o_ref: torch.Tensor, what="O"):
    d = (o_dev.float().cpu() - o_ref.float()).abs()
    assert torch.isfinite(o_dev.float()).all(), f"{what}: non-finite values"
    assert d.max().item() <= O_MAX_ABS, f"{what}: max-abs {d.max().item():.3e}"
    assert d.mean().item() <= O_MEAN_ABS, f"{what}: mean-abs {d.mean().item():.3e}"
    ref_norm = o_ref.float().norm().item()
    if ref_norm > 0:
        rel = (o_dev.float().cpu() - o_ref.float()).norm().item() / ref_norm
        assert rel <= GRAD_REL_L2, f"{what}: rel-L2 {rel:.3e}"


def check_lse(l_dev: torch.Tensor, l_ref: torch.Tensor, what="LSE"):
    l_dev = l_dev.float().cpu().reshape(l_ref.shape)
    inf_ref = torch.isinf(l_ref) & (l_ref < 0)
    inf_dev = torch.isinf(l_dev) & (l_dev < 0)
    assert torch.equal(inf_ref, inf_dev), f"{what}: -inf rows differ"
    fin = ~inf_ref
    if fin.any():
        d = (l_dev[fin] - l_ref[fin]).abs().max().item()
        assert d <= LSE_ABS, f"{what}: max-abs {d:.3e}"


def check_grad(g_dev: torch.Tensor, g_ref: torch.Tensor, what="grad"):
    g = g_dev.float().cpu()
    r = g_ref.float()
    assert torch.isfinite(g).all(), f"{what}: non-finite values"
    scale = max(r.abs().max().item(), 1e-30)
    d = (g - r).abs()
    assert d.max().item() <= O_MAX_ABS * scale, f"{what}: max-abs {d.max().item():.3e} vs scale {scale:.3e}"
    assert d.mean().item() <= O_MEAN_ABS * scale, f"{what}: mean-abs {d.mean().item():.3e} vs scale {scale:.3e}"
    rn = r.norm().item()
    if rn > 0:
        rel = (g - r).norm().item() / rn
        assert rel <= GRAD_REL_L2, f"{what}: rel-L2 {rel:.3e}"
