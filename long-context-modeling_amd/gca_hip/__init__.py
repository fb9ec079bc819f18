"""MI355X-native Grouped Cross-Attention and landmark retrieval (HIP kernels behind a C ABI)."""
from . import _lib
from .gca import attention, gca_kv_cache, attention_indexed, gca_kv_cache_indexed, attention_tokens, list_cache
from .retrieval import (landmark_scores, landmark_topk, landmark_score_topk, landmark_retrieve,
                        landmark_retrieve_static, gather_chunks, gca_layer)
from .chunk_cache import ChunkKVManager, chunk_cache_append
from .module import GroupCrossAttention

__all__ = [
    "attention", "gca_kv_cache", "attention_indexed", "gca_kv_cache_indexed",
    "landmark_scores", "landmark_topk", "landmark_score_topk", "landmark_retrieve", "landmark_retrieve_static", "gather_chunks", "gca_layer",
    "ChunkKVManager", "chunk_cache_append", "attention_tokens", "GroupCrossAttention",
]
