"""Hugging Face integration for Llama-3.2-Vision (Mllama) cross-attention.

The reference replaces `MllamaTextCrossSdpaAttention.forward` of transformers
4.47 by hand (test_llama3.py:356-468, installed at :666-668).  Current
transformers releases route every attention layer through a pluggable
attention interface, so the same substitution is one registration:

    from lv_xattn.hf_mllama import register
    register()                                  # adds the "lv_xattn" implementation
    model.config._attn_implementation = "lv_xattn"      # or per sub-config

`MllamaTextCrossAttention.forward` then hands the projected, normalised
Q [B,Hq,Lq,D], K, V [B,Hkv,Lkv,D] and the additive cross-attention mask
[B,1,Lq,Lkv] to `lv_xattn_attention_forward`, which runs the gfx950 flash
forward / backward (dense-bias variant; K/V kept for backward, as in the
reference's `create_attention_class_save_qkv`, test_llama3.py:125-178).
The registry is model-wide, so the causal self-attention layers arrive here as
well; they are not this operator and are passed on to transformers' own
implementation.  A cross-attention call the kernels do not cover (not bf16 on
the GPU, head_dim other than 16, 32, 64 or 128 (the patched layer forward: 128), dropout) raises.

`patch_cross_attention_forward(model)` goes one step further, like the
reference's recompute variant (`create_attention_class`,
test_llama3.py:180-245, used by the patched forward at :361-466): the K/V
projections and the k_norm move inside the autograd function, so K and V are
not kept between forward and backward but recomputed from the visual hidden
states by the gfx950 GEMM (norm fused in its epilogue).
"""
from __future__ import annotations

from typing import Optional

import torch

from ._lib import LvxError
from .autograd import create_attention_class, create_attention_class_save_qkv, create_q_projection_class

NAME = "lv_xattn"
_attention = None
_bias_cache: list = []      # [key, fp32 bias, the mask it was made from] of the last conversion


def _mask_bias(mask: torch.Tensor) -> torch.Tensor:
    """transformers fills masked positions with the dtype's most negative finite
    value (-3.4e38 in bf16).  The kernels add the bias to the fp32 scores and, in
    backward, subtract the row's LSE from score + bias, so the fill value is
    limited to -30000: exp(-30000) is still exactly 0 next to any visible key,
    and the subtraction stays accurate.  A row that is masked everywhere then
    attends by its scores over the masked keys (as it does in the reference,
    whose fp16 fill value is -65504; transformers' eager path attends uniformly
    there).  The masks transformers builds hold no such row: its
    _prepare_cross_attention_mask multiplies the mask by
    full_text_row_masked_out_mask, which turns a row that sees no tile into a
    row that sees every key.
    Where a row does see a key, its masked positions become -inf: the result is the same
    (exp(-30000) is already 0 there) and the kernels can then skip whole tiles outside the span
    of the visible keys (ops.bias_hull), which is most of a Llama-3.2 mask.  A converted mask that
    is kept is marked as such: the attention call then tests it once for being a pure interval
    mask (every row sees one run of keys, bias 0 there) and, when it is, runs without the bias."""
    # an inference tensor (torch.inference_mode) has no version counter: its contents cannot be told
    # apart from an edited copy at the same address, so it is converted every time and not kept
    version = None if mask.is_inference() else mask._version
    key = (mask.data_ptr(), version, tuple(mask.shape), tuple(mask.stride()), mask.dtype, mask.device)
    if version is not None and _bias_cache and _bias_cache[0] == key:
        return _bias_cache[1]
    m = mask.float()
    masked = m <= -30000.0
    sees_a_key = (~masked).any(-1, keepdim=True)
    bias = torch.where(masked & sees_a_key, float("-inf"), m.clamp_min(-30000.0))
    # every cross-attention layer of a model gets the same mask, in forward and again in backward:
    # the last conversion is kept (with the mask itself, so that its address cannot be reused)
    if version is not None:
        bias.lvx_reused = True      # attn._bias_and_hull: worth testing once whether it is an interval mask
        _bias_cache[:] = [key, bias, mask]
    return bias


def clear_mask_cache() -> None:
    """Drops the converted mask `_mask_bias` keeps (an fp32 tensor of the mask's size)."""
    _bias_cache.clear()


def lv_xattn_attention_forward(module, query, key, value, attention_mask: Optional[torch.Tensor],
                               dropout: float = 0.0, scaling: Optional[float] = None, **kwargs):
    """Attention-interface function (same contract as transformers'
    eager_attention_forward): returns (attn_output [B, Lq, Hq, D], None)."""
    global _attention
    if kwargs.get("is_causal", False) or getattr(module, "is_causal", False) is True or not hasattr(module, "k_norm"):
        # a (causal) self-attention layer: another operator, transformers' own.  Its SDPA
        # form, because the masks this implementation name is registered with (see register)
        # are SDPA masks: None stands for "plain causal", which eager attention would read
        # as "no mask at all".
        from transformers.integrations.sdpa_attention import sdpa_attention_forward
        return sdpa_attention_forward(module, query, key, value, attention_mask, dropout=dropout,
                                      scaling=scaling, **kwargs)
    _require_supported(query, key, dropout)
    if _attention is None:
        _attention = create_attention_class_save_qkv("lv_xattn", rounds=1, batched=True).apply
    if scaling is None:
        scaling = query.shape[-1] ** -0.5
    if attention_mask is None:
        out = _attention(query, key, value, False, scaling)
    else:
        Lq, Lkv = query.shape[2], key.shape[2]
        mask = attention_mask[..., :Lq, :Lkv]
        out = _attention(query, key, value, False, scaling, _mask_bias, [mask], [])
    return out.transpose(1, 2).contiguous(), None


def _require_supported(query, key, dropout):
    if not (query.is_cuda and query.dtype in (torch.bfloat16, torch.float16) and query.shape[-1] in (16, 32, 64, 128) and dropout == 0.0
            and query.shape[1] % key.shape[1] == 0):
        raise LvxError("lv_xattn cross-attention needs bf16 or fp16 tensors on the GPU, head_dim 16, 32, 64 or 128, no dropout and "
                       f"Hkv | Hq; got {query.dtype} on {query.device}, q {tuple(query.shape)}, "
                       f"k {tuple(key.shape)}, dropout {dropout}")


_recompute = {}


def _recompute_forward(self, hidden_states, cross_attention_states=None, past_key_values=None,
                       attention_mask=None, use_cache=None, **kwargs):
    """Replacement for MllamaTextCrossAttention.forward with the K/V recompute
    of the reference's patched forward (test_llama3.py:361-466).  Extra
    keyword `lvx_mask`: a compact `Mask` (see mask_from_cross_attention_mask)
    used instead of the dense `attention_mask`."""
    if cross_attention_states is None or past_key_values is not None:
        # decoding from a K/V cache: nothing to recompute; the stock forward
        # still reaches the kernels through the attention interface
        return self._lvx_stock_forward(hidden_states, cross_attention_states, past_key_values,
                                       attention_mask, use_cache, **kwargs)
    bsz, q_len, _ = hidden_states.size()
    dropout = self.dropout if self.training else 0.0
    if not (hidden_states.is_cuda and hidden_states.dtype in (torch.bfloat16, torch.float16) and self.head_dim == 128
            and dropout == 0.0):
        raise LvxError("lv_xattn cross-attention needs bf16 or fp16 tensors on the GPU, head_dim 128 and no dropout")
    key = (self._lvx_rounds, self._lvx_batched, self._lvx_weight_grads)
    if key not in _recompute:
        _recompute[key] = create_attention_class("lv_xattn", rounds=key[0], batched=key[1],
                                                 weight_grads=key[2], w_in_major=False).apply
    if ("q", key[2]) not in _recompute:
        _recompute[("q", key[2])] = create_q_projection_class(w_in_major=False, weight_grads=key[2]).apply
    # q_proj + q_norm in the fused GEMM; like K/V, Q is recomputed from the layer input in backward
    query = _recompute[("q", key[2])](hidden_states.contiguous(), self.q_proj.weight, self.num_heads,
                                      self.q_norm.weight, self.q_norm.variance_epsilon)
    mask = kwargs.get("lvx_mask")
    bias = []
    if mask is None and attention_mask is not None:
        lkv = cross_attention_states.shape[1]
        bias = [_mask_bias, attention_mask[..., :q_len, :lkv]]
    out = _recompute[key](query, cross_attention_states.to(query.dtype), self.k_proj.weight, self.v_proj.weight,
                          self.num_key_value_heads, self.scaling, mask, self.k_norm.weight,
                          self.k_norm.variance_epsilon, *bias)
    out = out.transpose(1, 2).reshape(bsz, q_len, -1)
    return self.o_proj(out), None


def patch_cross_attention_forward(model, rounds: int = 1, batched: bool = True, weight_grads: bool = True) -> int:
    """Installs the recompute forward on every MllamaTextCrossAttention module
    under `model` (the reference assigns its patched forward to the class,
    test_llama3.py:666-668; here it is per instance, so unpatching is
    `del module.forward`).  Returns the number of modules patched."""
    import types
    from transformers.models.mllama.modeling_mllama import MllamaTextCrossAttention
    n = 0
    for mod in model.modules():
        if isinstance(mod, MllamaTextCrossAttention):
            mod._lvx_stock_forward = types.MethodType(MllamaTextCrossAttention.forward, mod)
            mod._lvx_rounds, mod._lvx_batched, mod._lvx_weight_grads = rounds, batched, weight_grads
            mod.forward = types.MethodType(_recompute_forward, mod)
            n += 1
    return n


def register() -> str:
    """Adds the implementation to transformers' attention registry and returns
    its name.  Raises ImportError if transformers has no attention interface."""
    from transformers import AttentionInterface
    AttentionInterface.register(NAME, lv_xattn_attention_forward)
    # The registry is model-wide: the self-attention layers get their masks by this name too.
    # Without an entry transformers builds no mask at all for a custom implementation (padding
    # included), so the name is given the SDPA mask builder.
    from transformers.masking_utils import AttentionMaskInterface, sdpa_mask
    AttentionMaskInterface.register(NAME, sdpa_mask)
    return NAME


def mask_from_cross_attention_mask(cross_attention_mask: torch.Tensor, num_vision_tokens: int,
                                   kv_len: Optional[torch.Tensor] = None, empty_rows: str = "all"):
    """Compact form of a Llama-3.2 cross-attention mask.

    `cross_attention_mask` is what the Mllama processor emits, [B, T, n_images,
    n_tiles] with 1 where text token t may look at that tile; every tile stands
    for `num_vision_tokens` consecutive keys, in (image, tile) order - the
    expansion transformers does in `_prepare_cross_attention_mask` before
    turning it into the dense additive bias the reference feeds to `bias_func`
    (lv_xattn/attn.py:386-389).  When every row's visible keys form one
    contiguous range (the usual case: a token looks at the tiles of the most
    recent image) this returns `Mask(kv_len, kv_start, kv_end)` for the interval
    kernels - 8 bytes per row instead of 4 bytes per (row, key).  Returns None if
    some row has a gap (e.g. unused tile slots between two visible images): use
    the dense bias then.

    A row that may look at no tile (text before the first image) follows
    `empty_rows`: "all" (default) lets it see every key, which is what
    `_prepare_cross_attention_mask` makes of it (it multiplies the additive mask
    by full_text_row_masked_out_mask) and hence what the dense bias of the
    reference holds; "none" gives it an empty interval (O = 0, LSE = -inf,
    dQ = 0)."""
    from .ops import Mask
    if empty_rows not in ("all", "none"):
        raise ValueError("empty_rows must be 'all' or 'none'")
    B, T = cross_attention_mask.shape[:2]
    vis = cross_attention_mask.reshape(B, T, -1) != 0              # [B, T, n_images * n_tiles]
    n = vis.shape[-1]
    idx = torch.arange(n, device=vis.device)
    any_vis = vis.any(-1)
    first = torch.where(vis, idx, n).amin(-1)
    last = torch.where(vis, idx, -1).amax(-1)
    count = vis.sum(-1)
    if not bool(((last - first + 1 == count) | ~any_vis).all()):
        return None
    empty_end = n if empty_rows == "all" else 0
    start = torch.where(any_vis, first, torch.zeros_like(first)) * num_vision_tokens
    end = torch.where(any_vis, last + 1, torch.full_like(last, empty_end)) * num_vision_tokens
    return Mask(None if kv_len is None else kv_len.to(torch.int32), start.to(torch.int32).contiguous(),
                end.to(torch.int32).contiguous())
