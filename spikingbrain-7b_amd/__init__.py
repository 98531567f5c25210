"""MI355X-native decode-time cache hot path of a SpikingBrain-7B-shaped hybrid model.

The directory name contains a hyphen, so it is loaded by path (see `__graft_entry__.load_package`)
and registered in `sys.modules` as `spikingbrain_7b_amd`.

  hf_cache.Cache                      drop-in for hf_7B_model/cache.py
  window_attention                    cache + attention slice of the HF sliding-window layer
  meta_attention.MetaAttention*       drop-in for vllm_hymeta/attention/meta_attention.py
  gla                                 GLA recurrent step + constant-size state cache
  block_manager.WindowBlockManager    window eviction / block recycling / slot mapping
  ops                                 tensor-level wrappers over the C ABI (include/sbcache.h)
  decode_driver.HybridDecodeCache     the 28-layer stack's cache work per generated token
"""
from . import (_native, block_manager, decode_driver, gla, hf_cache, meta_attention, ops, runner,  # noqa: F401
               window_attention)
from .block_manager import PAD_SLOT_ID, WindowBlockManager, compute_slot_mapping, compute_slot_mapping_start_idx  # noqa: F401
from .decode_driver import HybridDecodeCache  # noqa: F401
from .gla import (GLACacheManager, GLACacheParams, fused_chunk_gla, fused_recurrent_gla,  # noqa: F401
                  gla_prefill_packed, my_fused_recurrent_gla)
from .hf_cache import Cache  # noqa: F401
from .meta_attention import (AttentionType, Int8KVCache, MetaAttentionBackend, MetaAttentionImpl,  # noqa: F401
                             MetaAttentionMetadata, MetaAttentionMetadataBuilder)
from .runner import SwaCacheRunner  # noqa: F401
from .window_attention import sliding_window_attention  # noqa: F401

__all__ = [
    "Cache", "sliding_window_attention", "MetaAttentionBackend", "MetaAttentionImpl", "MetaAttentionMetadata",
    "MetaAttentionMetadataBuilder", "AttentionType", "Int8KVCache", "GLACacheManager", "GLACacheParams",
    "my_fused_recurrent_gla", "fused_recurrent_gla", "fused_chunk_gla", "gla_prefill_packed", "WindowBlockManager", "PAD_SLOT_ID",
    "compute_slot_mapping", "compute_slot_mapping_start_idx", "ops", "SwaCacheRunner", "HybridDecodeCache",
]
