"""Host-side logic that needs no GPU: block bounds, the transport shims, the
argument checks of the Python mirror of the reference API."""
import pytest
import torch

import lv_xattn
from lv_xattn import attn, ops
from lv_xattn import async_communication as ac
from oracle import lvx_oracle as orc


def test_public_names_match_reference_package():
    for name in ("_attn_forward", "_attn_backward", "initialize_distributed",
                 "reset_global_memory_buffer", "get_sequence_parallel_group"):
        assert hasattr(lv_xattn, name)


def test_block_bounds_agree_with_oracle():
    for lq, p in ((4096, 16), (3000, 16), (1777, 16), (10, 4), (5, 8)):
        assert attn.q_block_bounds(lq, p) == orc.q_block_bounds(lq, p)
        b = attn.q_block_bounds(lq, p)
        assert b[0][0] == 0 and b[-1][1] == lq
        assert all(b[i][1] == b[i + 1][0] for i in range(p - 1))


def test_round_group_shim(monkeypatch):
    monkeypatch.delenv("LVX_ROUNDS", raising=False)
    monkeypatch.setenv("WORLD_SIZE", "16")
    ac.initialize_distributed()
    g = lv_xattn.get_sequence_parallel_group()
    assert g.size() == 16 and g.rank() == 0
    ac.initialize_distributed(4)
    assert lv_xattn.get_sequence_parallel_group().size() == 4
    with pytest.raises(ValueError):
        ac.initialize_distributed(0)
    ac.initialize_distributed(3)
    assert ac.get_sequence_parallel_size() == 3 and ac.get_sequence_parallel_rank() == 0
    ac.destroy_sequence_parallel()
    assert ac.get_sequence_parallel_size() == 1


def test_workspace_cache_and_reset():
    lv_xattn.reset_global_memory_buffer()
    a = ac.workspace("t", (4, 4), torch.float32, "cpu")
    assert tuple(a.shape) == (4, 4) and a.dtype == torch.float32
    # one buffer per tag: the same memory for the same or a smaller request, whatever the shape ...
    assert ac.workspace("t", (4, 4), torch.float32, "cpu").data_ptr() == a.data_ptr()
    assert ac.workspace("t", (2, 3), torch.bfloat16, "cpu").data_ptr() == a.data_ptr()
    # ... grown (not multiplied) by a larger one
    b = ac.workspace("t", (64, 64), torch.float32, "cpu")
    assert tuple(b.shape) == (64, 64) and len(ac._WORKSPACES) == 1
    assert ac.workspace("t", (4, 4), torch.float32, "cpu").data_ptr() == b.data_ptr()
    assert ac.workspace("u", (4,), torch.float32, "cpu").data_ptr() != b.data_ptr() and len(ac._WORKSPACES) == 2
    lv_xattn.reset_global_memory_buffer()
    assert len(ac._WORKSPACES) == 0
    lv_xattn.reset_global_memory_buffer("lv_xattn")      # the reference passes the mode


def test_backward_row_windows_are_cut_to_the_workspace_cap():
    per_row = 2 * 8 * 32 * 6528                 # bytes of dS^T per text row at B8 Hq32 Lkv6404 (6528 = 51 x 128)
    nbytes = lambda rows: per_row * ((rows + 31) // 32 * 32) + (1 << 20)
    # under the cap: untouched
    assert attn._cap_windows([(0, 4096)], nbytes, 14 << 30) == [(0, 4096)]
    # over it: chunks of whole 256-row groups that fit, covering the window exactly
    cut = attn._cap_windows([(0, 4096)], nbytes, 4 << 30)
    assert cut[0][0] == 0 and cut[-1][1] == 4096 and all(a[1] == b[0] for a, b in zip(cut, cut[1:]))
    assert all(nbytes(r1 - r0) <= 4 << 30 and (r1 - r0) % 256 == 0 for r0, r1 in cut[:-1]) and len(cut) == 4
    # per-round windows that already fit stay as they are; a 256-row window is never cut
    assert attn._cap_windows([(0, 188), (188, 376)], nbytes, 1 << 30) == [(0, 188), (188, 376)]
    assert attn._cap_windows([(0, 256)], nbytes, 1 << 20) == [(0, 256)]
    with pytest.raises(ValueError):
        ac.set_backward_workspace_cap(1 << 20)


def test_causal_and_malformed_bias_are_rejected_explicitly():
    q = torch.zeros(1, 4, 8, 128, dtype=torch.bfloat16)
    k = torch.zeros(1, 2, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="causal"):
        lv_xattn._attn_forward(q, k, k, True, 0.1, None)
    with pytest.raises(ValueError, match="bias_func must return"):
        lv_xattn._attn_forward(q, k, k, False, 0.1, None, bias_func=lambda: torch.zeros(1, 1, 3, 8))
    with pytest.raises(ValueError, match="without a bias_func"):
        lv_xattn._attn_forward(q, k, k, False, 0.1, None, local_bias_args=[torch.zeros(1)])
    with pytest.raises(ValueError, match="causal"):
        lv_xattn._attn_backward(q, q, k, k, q, torch.zeros(4, 8), True, 0.1, None, "flash")
    # the reference's patched Mllama forward passes is_causal=True when there is no mask and
    # more than one query (test_llama3.py:430): the refusal says where that comes from, in the
    # round loops and in both autograd wrappers
    with pytest.raises(ValueError, match=r"test_llama3\.py:430"):
        lv_xattn._attn_forward(q, k, k, True, 0.1, None)
    with pytest.raises(ValueError, match=r"test_llama3\.py:430"):
        lv_xattn.create_attention_class_save_qkv("lv_xattn").apply(q, k, k, True, 0.1)
    with pytest.raises(ValueError, match=r"test_llama3\.py:430"):
        lv_xattn.create_attention_class("lv_xattn").apply(q, lambda x, vis: (q, k, k), True)


def test_shape_and_dtype_checks_raise_before_any_device_call():
    q = torch.zeros(1, 4, 8, 128, dtype=torch.float32)
    k = torch.zeros(1, 2, 8, 128, dtype=torch.float32)
    with pytest.raises(ops.LvxError, match="bf16 or fp16"):
        ops._shape(q, k, 0.1, None)
    with pytest.raises(ops.LvxError, match="one type"):          # q and k of different 16-bit types
        ops._shape(q.half(), k.bfloat16(), 0.1, None)
    assert ops._shape(q.half(), k.half(), 0.1, None).dtype == 2 and ops._shape(q.bfloat16(), k.bfloat16(), 0.1, None).dtype == 1
    qb, kb = q.bfloat16(), torch.zeros(2, 2, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(ops.LvxError, match="disagree"):
        ops._shape(qb, kb, 0.1, None)
    kb = torch.zeros(1, 2, 8, 128, dtype=torch.bfloat16)
    bad = ops.Mask(kv_len=torch.zeros(3, dtype=torch.int32))
    with pytest.raises(ops.LvxError, match="kv_len"):
        ops._shape(qb, kb, 0.1, bad)
    with pytest.raises(ops.LvxError, match="unit last stride"):
        ops.t4(torch.zeros(1, 2, 128, 8, dtype=torch.bfloat16).transpose(2, 3))


def test_llama_cross_attention_mask_to_intervals():
    from lv_xattn.hf_mllama import mask_from_cross_attention_mask
    # 2 samples, 6 text tokens, 2 images x 4 tile slots, 5 keys per tile
    cam = torch.zeros(2, 6, 2, 4, dtype=torch.int64)
    cam[0, 1:4, 0, :2] = 1          # tokens 1-3 see tiles 0,1 of image 0
    cam[0, 4:, 1, :] = 1            # tokens 4-5 see all four tiles of image 1
    cam[1, 2:, 0, :4] = 1           # sample 1: tokens 2.. see image 0 (4 tiles) ...
    cam[1, 5, 1, :1] = 1            # ... and token 5 also tile 0 of image 1 (adjacent: still one range)
    m = mask_from_cross_attention_mask(cam, 5, empty_rows="none")
    assert m is not None and m.kv_start.dtype == torch.int32
    assert m.kv_start.tolist() == [[0, 0, 0, 0, 20, 20], [0, 0, 0, 0, 0, 0]]
    assert m.kv_end.tolist() == [[0, 10, 10, 10, 40, 40], [0, 0, 20, 20, 20, 25]]
    # the dense expansion says the same
    dense = cam.reshape(2, 6, 8).repeat_interleave(5, dim=-1).bool()
    k = torch.arange(40)
    assert torch.equal(dense, (k >= m.kv_start[..., None]) & (k < m.kv_end[..., None]))
    # default: rows that may look at no tile see every key, which is what transformers' own
    # mask preparation makes of them
    from transformers.models.mllama.modeling_mllama import _prepare_cross_attention_mask
    m = mask_from_cross_attention_mask(cam, 5)
    assert m.kv_end.tolist() == [[40, 10, 10, 10, 40, 40], [40, 40, 20, 20, 20, 25]]
    hf_mask, _ = _prepare_cross_attention_mask(cam.float(), 5, torch.float32)       # [B, 1, T, keys], 0 = visible
    assert torch.equal(hf_mask[:, 0] == 0, (k >= m.kv_start[..., None]) & (k < m.kv_end[..., None]))
    # a gap (image 0 with 2 of 4 tiles, then image 1) has no interval form
    cam[0, 5, 0, :2] = 1
    assert mask_from_cross_attention_mask(cam, 5) is None


def test_bench_refuses_more_than_one_gpu():
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "single-GPU" in (r.stderr + r.stdout)


def test_mask_conversion_of_the_hf_hook_under_inference_mode():
    """An inference tensor has no version counter: the converted mask is then rebuilt on every call
    instead of being kept, and no error is raised."""
    from lv_xattn import hf_mllama
    hf_mllama.clear_mask_cache()
    neg = torch.finfo(torch.bfloat16).min
    with torch.inference_mode():
        mask = torch.zeros(1, 1, 3, 8, dtype=torch.bfloat16)
        mask[0, 0, 1, 4:] = neg
        b1 = hf_mllama._mask_bias(mask)
        assert b1.dtype == torch.float32 and b1[0, 0, 1, 4:].eq(float("-inf")).all() and b1[0, 0, 1, :4].eq(0).all()
        mask[0, 0, 2, :2] = neg                   # edited in place: no version tells, so nothing may be reused
        b2 = hf_mllama._mask_bias(mask)
        assert b2[0, 0, 2, :2].eq(float("-inf")).all()
    assert not hf_mllama._bias_cache
    # an ordinary tensor is kept until it changes
    mask = torch.zeros(1, 1, 3, 8, dtype=torch.bfloat16)
    assert hf_mllama._mask_bias(mask) is hf_mllama._mask_bias(mask)
    mask[0, 0, 0, 0] = neg
    assert hf_mllama._mask_bias(mask)[0, 0, 0, 0] == float("-inf")
    hf_mllama.clear_mask_cache()
