"""MI355X-native OMMX paged decode-attention path (store, split-KV decode, combine)."""
__version__ = "0.1.0"

from .attention import (WindowSpec, ommx_pack_kv_canonical_block,  # noqa: F401
                        ommx_paged_decode_attention_canonical, store_pack_into)
