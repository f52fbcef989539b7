"""vesper_amd: MI355X-native attention hot path (prefill, KV-cache decode, KV append) behind the
reference's operator surface.  The compute lives in lib/libvsp_attn.so (HIP, gfx950, C ABI in
include/vsp_attn.h); this package is the thin Python view of it used by tests and bench.py.
The C++ mirror of the reference's interfaces is in csrc/adapter/."""
from . import _ffi  # noqa: F401  (raises if the HIP library is missing)
from .api import (KVCache, GQAKVCache, RaggedKVCache, RopeTable, VspError, attention_core, decode_attention, decode_attention_multi, decode_attention_noalloc, decode_attention_proj, flash_attention, flash_attention_split,
                  flash_attention_backward, flash_attention_backward_split, backward_workspace,
                  repeat_kv_is_fused, scaled_dot_product_attention)

__all__ = ["KVCache", "GQAKVCache", "RaggedKVCache", "RopeTable", "VspError", "attention_core", "decode_attention", "decode_attention_multi", "decode_attention_noalloc", "decode_attention_proj", "flash_attention", "flash_attention_split",
           "flash_attention_backward", "flash_attention_backward_split", "backward_workspace",
           "repeat_kv_is_fused", "scaled_dot_product_attention"]
