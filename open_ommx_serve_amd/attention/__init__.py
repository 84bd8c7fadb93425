"""OMMX paged decode attention on AMD gfx950: store, decode and window arithmetic.

The public names mirror ``ommx_gpu_serve.attention`` of the reference.
"""
from .kv_pool import MultiSeqKVPool
from .kv_store import CanonicalKVStore
from .kv_store_ops import gather_tail, gather_tails, ring_slot, write_token, write_tokens
from .kv_window import WindowSpec, packed_boundary, tail_token_indices
from .pack import (CANONICAL_GROUP_CHANNELS, CANONICAL_GROUP_TOKENS, alloc_planes,
                   ommx_pack_kv_canonical_block, store_pack_into)
from .paged_decode import (auto_num_kv_splits, make_attn_logits, merge_attention_states,
                           ommx_paged_decode_attention_canonical)

__all__ = [
    "ommx_paged_decode_attention_canonical", "ommx_pack_kv_canonical_block", "store_pack_into",
    "alloc_planes", "auto_num_kv_splits", "make_attn_logits", "WindowSpec", "packed_boundary",
    "tail_token_indices", "CANONICAL_GROUP_TOKENS", "CANONICAL_GROUP_CHANNELS",
    "MultiSeqKVPool", "CanonicalKVStore", "write_token", "write_tokens", "gather_tail",
    "gather_tails", "ring_slot", "merge_attention_states",
]
