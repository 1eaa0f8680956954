"""MI355X-native paged-KV attention path behind FastDeploy's attention op surface.

Host code is Python; the kernels are hand-written HIP for gfx950 reached through
the C ABI of libfdattn.so (include/fdattn.h) with ctypes.  torch tensors are used
only as device buffers.
"""
from .ops import (  # noqa: F401
    append_attention,
    append_attention_workspace,
    append_attention_prefill,
    decode_attention,
    decode_attention_sparse,
    decode_uses_mfma,
    decode_workspace,
    prefill_auto_splits,
    splitkv_combine,
    sqattn_select,
    write_cache_kv,
)
from .backend import AppendAttentionBackend, AttentionLayer, ForwardMeta, SequenceBook  # noqa: F401
from .block_pool import BlockPool  # noqa: F401
from .rope import rope_table  # noqa: F401

__version__ = "0.1"
