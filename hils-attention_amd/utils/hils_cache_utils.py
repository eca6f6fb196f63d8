"""KV cache of one HiLS layer for decoding, with the pooled chunk keys kept up to date.

The reference keeps the cache in ``HiLSDynamicLayer`` (utils/hils_cache_utils.py:8-76), which
re-concatenates K and V on every step, and the pooled chunk keys in ``_hils_prior_cache``
(models/FlashHiLS/hils_attention.py:361-416), extended whenever a chunk fills.  Here the three
tensors are allocated once at a capacity and written in place: the selection only looks at chunks
the causal limit makes visible (``q_offset``), so the kernels can be handed the whole buffers and
no tensor is copied or re-laid-out per step.  Mean-pooled chunk keys only (the layer's
``enable_chunk_pooling`` mode)."""
import math

import torch

try:  # imported as part of the package ...
    from ..ops.chunk_attn_pool_tilelang import chunk_mean_pool
    from ..ops.hils_fwd_bwd_head import HiLS_block_M_head
    from ..ops.hils_glue import topk_chunk_weights
except ImportError:  # ... or with the package directory itself on sys.path (`from utils... import`)
    from ops.chunk_attn_pool_tilelang import chunk_mean_pool
    from ops.hils_fwd_bwd_head import HiLS_block_M_head
    from ops.hils_glue import topk_chunk_weights


class HiLSDynamicLayer:
    """update() / get_seq_length() as in the reference's class; the buffers grow by doubling."""

    is_sliding = False

    def __init__(self, chunk_size=64, capacity=0):
        self.chunk_size = int(chunk_size)
        self.capacity = int(capacity)
        self.seq_len = 0
        self.pooled_chunks = 0  # chunks whose mean-pooled key is in lmk_k
        self.keys = self.values = self.lmk_k = None
        self.is_initialized = False

    def lazy_initialization(self, key_states, value_states):
        B, T, H, D = key_states.shape
        S = self.chunk_size
        cap = max(self.capacity, T, S)
        cap = (cap + S - 1) // S * S
        self.capacity = cap
        self.dtype, self.device = key_states.dtype, key_states.device
        self.keys = torch.empty((B, cap, H, D), dtype=self.dtype, device=self.device)
        self.values = torch.empty((B, cap, H, value_states.shape[-1]), dtype=self.dtype, device=self.device)
        self.lmk_k = torch.zeros((B, cap // S, H, D), dtype=self.dtype, device=self.device)
        self.is_initialized = True

    def _grow(self, need):
        S = self.chunk_size
        cap = self.capacity
        while cap < need:
            cap *= 2
        cap = (cap + S - 1) // S * S
        for name in ("keys", "values", "lmk_k"):
            old = getattr(self, name)
            rows = cap // S if name == "lmk_k" else cap
            new = torch.zeros((old.shape[0], rows) + tuple(old.shape[2:]), dtype=old.dtype, device=old.device)
            new[:, : old.shape[1]] = old
            setattr(self, name, new)
        self.capacity = cap

    def update(self, key_states, value_states, *args, **kwargs):
        """Append (B, T, H, D) keys / values; pool the chunks they complete.  Returns views of the
        valid part of the cache (what the reference's update returns)."""
        if not self.is_initialized:
            self.lazy_initialization(key_states, value_states)
        T = key_states.shape[1]
        if self.seq_len + T > self.capacity:
            self._grow(self.seq_len + T)
        a, b = self.seq_len, self.seq_len + T
        self.keys[:, a:b] = key_states
        self.values[:, a:b] = value_states
        self.seq_len = b
        S = self.chunk_size
        full = b // S
        if full > self.pooled_chunks:
            c0 = self.pooled_chunks
            self.lmk_k[:, c0:full] = chunk_mean_pool(self.keys[:, c0 * S: full * S].contiguous(), S)
            self.pooled_chunks = full
        return self.keys[:, :b], self.values[:, :b]

    def get_seq_length(self):
        return self.seq_len

    def get_mask_sizes(self, query_length):
        return self.seq_len + query_length, 0

    def get_max_cache_shape(self):
        return -1

    def hils_attend(self, q, lse_swa, topk, window_size, sm_scale=None):
        """The remote (HiLS) branch for the last ``q.shape[1]`` positions of the cache: chunk
        selection, inter-chunk softmax and sparse attention on the cache buffers in place.
        q (B, Lq, h_q, D) bf16, lse_swa (B, Lq, h_q) of the local branch.  Returns
        (o_remote (B, Lq, h_q, Dv), weights (B, Lq, h_q, topk + 1), indices); the layer adds
        ``swa_o * weights[..., topk]`` to o_remote."""
        assert self.is_initialized and q.shape[1] <= self.seq_len
        S = self.chunk_size
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(q.shape[-1])
        idx, _, w = topk_chunk_weights(q, self.lmk_k, lse_swa, topk, S, window_size,
                                       q_offset=self.seq_len - q.shape[1], sm_scale=sm_scale)
        o = HiLS_block_M_head(q, self.keys, self.values, w, idx, block_size=S, sm_scale=sm_scale,
                              is_training=False)
        return o, w, idx
