"""MI355X-native drop-in for the `lv_xattn` attention API.

Same public names as the reference package (lv_xattn/__init__.py:1-2 there);
device work is done by hand-written gfx950 kernels in liblvx.so.
"""
from .attn import _attn_forward, _attn_backward, Mask, q_block_bounds
from .async_communication import (initialize_distributed, reset_global_memory_buffer,
                                  get_sequence_parallel_group)
from .autograd import (create_attention_class, create_attention_class_save_qkv, create_q_projection_class,
                       create_kv_projection_class, KVProjection, set_global_cross_attention_states,
                       get_global_cross_attention_states, clear_global_cross_attention_states)

__all__ = [
    "_attn_forward", "_attn_backward", "initialize_distributed", "reset_global_memory_buffer",
    "get_sequence_parallel_group", "Mask", "q_block_bounds",
    "create_attention_class", "create_attention_class_save_qkv", "create_q_projection_class",
    "create_kv_projection_class", "KVProjection", "set_global_cross_attention_states",
    "get_global_cross_attention_states", "clear_global_cross_attention_states",
]
