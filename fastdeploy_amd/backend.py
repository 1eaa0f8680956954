"""Attention backend: the caller's side of the path.  One object per model holds what every layer
shares (shapes, rotation table, workspace); per step the caller fills a ForwardMeta with the batch's
sequence lengths and block table, calls init_attention_metadata once, then forward_mixed once per layer.

The split follows the way the reference drives a backend: set-up once, bind tensors, run
(fastdeploy/runtime/runtime.h:48-104 Init / BindInputTensor / Infer), and its option object carrying
the static configuration (fastdeploy/runtime/runtime_option.h:34-60).
"""
from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import torch

from . import ops
from .block_pool import BlockPool


@dataclass
class AttentionLayer:
    """Per-layer constants: the layer's caches, their scales and the optional projection epilogue."""
    key_cache: torch.Tensor                      # uint8 / int8 / fp8 [num_blocks, kv_num_heads, block_size, head_dim]
    value_cache: torch.Tensor
    cache_k_scale: torch.Tensor                  # float32 [kv_num_heads, head_dim]; the dynamic formats: the scale
    cache_v_scale: torch.Tensor                  # caches [num_blocks, kv_num_heads, block_size] the cache writer fills
    qkv_bias: Optional[torch.Tensor] = None
    q_norm_weight: Optional[torch.Tensor] = None
    k_norm_weight: Optional[torch.Tensor] = None
    rms_norm_eps: float = 1e-6


@dataclass
class ForwardMeta:
    """One step's batch description (device int32 tensors, one entry per sequence slot)."""
    seq_lens_encoder: torch.Tensor               # > 0: a prefill row with that many new tokens
    seq_lens_decoder: torch.Tensor               # tokens already cached
    seq_lens_this_time: torch.Tensor             # new tokens of this step (0: idle slot)
    block_tables: torch.Tensor                   # [slots, max_blocks_per_seq]
    max_enc_len_this_time: Optional[int] = None  # host-side bound on seq_lens_encoder (0: no prefill row); found with one sync if None
    cu_seqlens_q: Optional[torch.Tensor] = None  # filled by init_attention_metadata
    num_tokens: int = 0                          # filled by init_attention_metadata
    prefill_rows: Optional[int] = None           # exact count of rows with seq_lens_encoder > 0, if known (None: unknown)
    prefill_splits: int = 1                      # filled by init_attention_metadata
    max_len_after: Optional[int] = None          # host-side: the longest sequence after this step (cached + new), if known;
                                                 # checked against the rotation table (positions past it are skipped by the writer)
    decode_tokens: int = 1                       # > 1: rows with seq_lens_encoder 0 and up to this many tokens
                                                 # (speculative drafts) are decode rows, one decode pass for all
    extra: dict = field(default_factory=dict)


class AppendAttentionBackend:
    def __init__(self, num_heads, kv_num_heads, head_dim, *, block_size=64, max_position=8192, rope_theta=10000.0,
                 rope_style="neox", cache_quant_type="cache_int8", softmax_scale=None, device="cuda",
                 sqattn_top_k=None, sqattn_per_token=False):
        from .rope import rope_table
        if num_heads % kv_num_heads:
            raise ValueError("num_heads %d is not a multiple of kv_num_heads %d" % (num_heads, kv_num_heads))
        self.num_heads, self.kv_num_heads, self.head_dim = num_heads, kv_num_heads, head_dim
        self.block_size, self.rope_style, self.cache_quant_type = block_size, rope_style, cache_quant_type
        self.softmax_scale = softmax_scale
        self.sqattn_top_k = sqattn_top_k   # > 0: decode rows attend to their top-k blocks only (block-sparse)
        # block-sparse decode rows of several tokens: one list per row (False) or one per token (True)
        self.sqattn_per_token = bool(sqattn_per_token)
        self.device = device
        self.rotary_embs = rope_table(max_position, head_dim, rope_theta, device)
        self._workspace = None
        self._out = None

    # ---- cache allocation -------------------------------------------------------------------------------
    def allocate_layer(self, num_blocks, cache_k_scale=None, cache_v_scale=None, **epilogue):
        """Zeroed caches of one layer ([num_blocks, kv_num_heads, block_size, head_dim] bytes each).  The per-channel
        formats need their scales (float32 [kv_num_heads, head_dim]); the dynamic formats get scale caches
        ([num_blocks, kv_num_heads, block_size], ones) that the cache writer fills row by row, the per-block formats
        scale caches [num_blocks, kv_num_heads] that it keeps tile by tile."""
        from .ops import is_dynamic, scale_cache_shape
        shape = (num_blocks, self.kv_num_heads, self.block_size, self.head_dim)
        kc = torch.zeros(shape, dtype=torch.uint8, device=self.device)
        vc = torch.zeros(shape, dtype=torch.uint8, device=self.device)
        if is_dynamic(self.cache_quant_type):
            if cache_k_scale is not None or cache_v_scale is not None:
                raise ValueError("the dynamic and per-block cache formats take no scales: the cache writer computes them")
            sshape = scale_cache_shape(self.cache_quant_type, num_blocks, self.kv_num_heads, self.block_size)
            cache_k_scale = torch.ones(sshape, dtype=torch.float32, device=self.device)
            cache_v_scale = torch.ones(sshape, dtype=torch.float32, device=self.device)
        elif cache_k_scale is None or cache_v_scale is None:
            raise ValueError("cache_k_scale and cache_v_scale are required for %r" % (self.cache_quant_type,))
        return AttentionLayer(kc, vc, cache_k_scale.to(self.device).contiguous(),
                              cache_v_scale.to(self.device).contiguous(), **epilogue)

    @staticmethod
    def blocks_for_memory(num_bytes, num_layers, kv_num_heads, head_dim, block_size=64):
        """How many blocks per layer fit into num_bytes of cache memory (K and V, one byte per value; the dynamic
        formats' scale caches add 4 bytes per stored row, 1/32 more at head_dim 128)."""
        per_block = 2 * kv_num_heads * block_size * head_dim * num_layers
        return int(num_bytes // per_block)

    # ---- per step ---------------------------------------------------------------------------------------
    def init_attention_metadata(self, meta: ForwardMeta):
        """Derives what the kernels need from the batch description: token offsets of the sequences,
        the token count and the bound on a prefill row's tokens; sizes the shared workspace."""
        this = meta.seq_lens_this_time
        if this.dtype != torch.int32 or not this.is_cuda:
            raise ValueError("seq_lens_this_time must be a device int32 tensor")
        slots = this.numel()
        if meta.block_tables.shape[0] != slots:
            raise ValueError("block_tables has %d rows, the batch %d slots" % (meta.block_tables.shape[0], slots))
        if meta.max_len_after is not None and meta.max_len_after > self.rotary_embs[0].shape[0]:
            raise ValueError("a sequence reaches %d tokens in this step, the rotation table holds %d positions "
                             "(max_position)" % (meta.max_len_after, self.rotary_embs[0].shape[0]))
        meta.cu_seqlens_q = ops.cu_seqlens_of(this)
        per_token = self.sqattn_per_token and (self.sqattn_top_k or 0) > 0 and meta.decode_tokens > 1
        if meta.decode_tokens > 1 and not per_token:
            group = self.num_heads // self.kv_num_heads
            if meta.decode_tokens * group > 16 or self.head_dim not in (64, 128, 256):
                raise ValueError("decode rows of %d tokens need head_dim 64, 128 or 256 and tokens x heads per KV head "
                                 "<= 16 (here %d): schedule such rows as prefill rows instead"
                                 % (meta.decode_tokens, meta.decode_tokens * group))
        if meta.max_enc_len_this_time is None:
            both = torch.stack([meta.cu_seqlens_q[-1], meta.seq_lens_encoder.max()]).tolist()   # one synchronisation
            meta.num_tokens, meta.max_enc_len_this_time = int(both[0]), max(int(both[1]), 0)
        elif meta.num_tokens <= 0:
            meta.num_tokens = int(meta.cu_seqlens_q[-1])
        # a step whose few prefill rows would leave CUs idle shares every query tile's keys among several workgroups
        meta.prefill_splits = 1
        if meta.prefill_rows and meta.max_enc_len_this_time > 0:
            meta.prefill_splits = ops.prefill_auto_splits(meta.prefill_rows, self.num_heads, meta.max_enc_len_this_time,
                                                           self.kv_num_heads)
        need = ops.append_attention_workspace_bytes(meta.num_tokens, slots * meta.decode_tokens if per_token else slots,
                                                    self.num_heads, self.kv_num_heads,
                                                    self.head_dim, meta.block_tables.shape[1], meta.prefill_splits)
        if self._workspace is None or self._workspace.numel() < need:
            self._workspace = torch.empty(need, dtype=torch.uint8, device=self.device)
        return meta

    def forward_mixed(self, qkv, layer: AttentionLayer, meta: ForwardMeta, out=None):
        """One layer's attention for the step described by meta: qkv bf16 [num_tokens, (H + 2 Hkv) D]
        -> bf16 [num_tokens, H D].  Writes the new tokens into the layer's caches."""
        if meta.cu_seqlens_q is None:
            raise ValueError("call init_attention_metadata(meta) first")
        if qkv.shape[0] != meta.num_tokens:
            raise ValueError("qkv has %d rows, the step %d tokens" % (qkv.shape[0], meta.num_tokens))
        return ops.append_attention(
            qkv, layer.key_cache, layer.value_cache, meta.seq_lens_encoder, meta.seq_lens_decoder,
            meta.seq_lens_this_time, meta.block_tables, self.rotary_embs, layer.cache_k_scale, layer.cache_v_scale,
            num_heads=self.num_heads, kv_num_heads=self.kv_num_heads, max_chunk=meta.max_enc_len_this_time,
            rope_style=self.rope_style, cache_quant_type=self.cache_quant_type, softmax_scale=self.softmax_scale,
            cu_seqlens_q=meta.cu_seqlens_q, workspace=self._workspace, out=out, qkv_bias=layer.qkv_bias,
            q_norm_weight=layer.q_norm_weight, k_norm_weight=layer.k_norm_weight, rms_norm_eps=layer.rms_norm_eps,
            prefill_rows=meta.prefill_rows, sqattn_top_k=self.sqattn_top_k, decode_tokens=meta.decode_tokens,
            sqattn_per_token=self.sqattn_per_token)


class SequenceBook:
    """Host-side bookkeeping of the sequence slots between steps: lengths, the block pool, and the
    ForwardMeta of the next step.  `schedule` takes the new tokens per slot ({slot: count}) - a count
    above one, or any count for an empty slot, makes a prefill row, unless the slot is named in `drafts`: its
    tokens are then the draft tokens of a speculative step and the row is a decode row of several tokens -
    reserves blocks and returns the meta; `commit` advances the lengths after the step has been enqueued (by the
    accepted count for a slot whose drafts were partly rejected: the next step overwrites the rest).  A reservation that fails (ValueError: the
    pool is exhausted or a table row is full) leaves the slots reserved earlier in the same call with their
    blocks: finish a sequence or retry with fewer tokens."""

    def __init__(self, pool: BlockPool, device="cuda", max_position=None):
        """max_position: the length of the backend's rotation table, if lengths are to be checked against it here."""
        self.pool, self.device, self.max_position = pool, device, max_position
        self.lengths = [0] * pool.max_seqs
        self._pending = None

    def schedule(self, new_tokens: dict, drafts=()) -> ForwardMeta:
        slots = self.pool.max_seqs
        enc, dec, this = [0] * slots, list(self.lengths), [0] * slots
        decode_tokens = 1
        for s, n in new_tokens.items():
            if n <= 0:
                continue
            if self.max_position is not None and self.lengths[s] + n > self.max_position:
                raise ValueError("slot %d would reach %d tokens, max_position is %d" % (s, self.lengths[s] + n, self.max_position))
            self.pool.reserve(s, self.lengths[s] + n)          # all or nothing per slot; raises when the pool is full
            this[s] = n
            if s in drafts and self.lengths[s] > 0:
                decode_tokens = max(decode_tokens, n)
            elif n > 1 or self.lengths[s] == 0:
                enc[s] = n
        i32 = lambda v: torch.tensor(v, dtype=torch.int32).to(self.device)
        self._pending = this
        return ForwardMeta(i32(enc), i32(dec), i32(this), self.pool.block_tables_tensor(self.device),
                           max_enc_len_this_time=max(enc), num_tokens=sum(this),
                           prefill_rows=sum(1 for n in enc if n > 0), decode_tokens=decode_tokens,
                           max_len_after=max(d + n for d, n in zip(dec, this)))

    def commit(self, accepted=None):
        """accepted: {slot: tokens of this step that stay} for speculative rows whose later drafts were rejected."""
        for s, n in enumerate(self._pending or []):
            keep = n if accepted is None or s not in accepted else accepted[s]
            if not 0 <= keep <= n:
                raise ValueError("slot %d: %d of %d tokens accepted" % (s, keep, n))
            self.lengths[s] += keep
        self._pending = None

    def finish(self, slot):
        self.pool.release(slot)
        self.lengths[slot] = 0

    def fork(self, src, dst):
        """Slot dst continues from the whole blocks of src's prefix; returns the tokens it inherited."""
        shared = self.pool.fork(src, dst, self.lengths[src])
        self.lengths[dst] = shared
        return shared
