"""DRAM Attention for AMD Instinct MI355X (gfx950): the reference package's
Python surface on hand-written HIP kernels (libdramattn.so)."""

__version__ = "0.1.0"

from .dram_attention import DRAMAttention, decode_attention
from .layer_stack import AttentionStack
from .kv_file import layer_cache_path, load_layer_cache, save_layer_cache
from .lru_cache import CacheOutput, DummyCache, LRUCache
from .lru_kernel import load_lru_cache_
from .max_ip_kernel import max_inner_product, max_ip_ref
from .topk_selector import IPUpperboundTopKSelector

__all__ = (
    "AttentionStack",
    "CacheOutput",
    "DRAMAttention",
    "DummyCache",
    "IPUpperboundTopKSelector",
    "LRUCache",
    "decode_attention",
    "layer_cache_path",
    "load_layer_cache",
    "load_lru_cache_",
    "max_inner_product",
    "max_ip_ref",
    "save_layer_cache",
)
