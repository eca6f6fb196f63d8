"""KV cache of one HiLS layer for decoding, with the pooled chunk keys kept up to date.

The reference keeps the cache in ``HiLSDynamicLayer`` (utils/hils_cache_utils.py:8-76), which
re-concatenates K and V on every step, and the per-chunk keys with their prior bias in
``_hils_prior_cache`` (models/FlashHiLS/hils_attention.py:361-416), extended whenever a chunk fills.
Here the tensors are allocated once at a capacity and written in place: the selection only looks at
chunks the causal limit makes visible (``q_offset``), so the kernels can be handed the whole buffers
and no tensor is copied or re-laid-out per step.  The chunk keys (and the prior bias) are kept
head-major, (B, H, chunks, D): the keys one (sequence, KV head) row of a decode step streams are
one contiguous block.  Both of the layer's modes: mean-pooled keys (``enable_chunk_pooling``) and,
given the chunks' prior queries ``mu_q``, the attention-pooled prior (``enable_prior_query``: entropy
bias per chunk and head, used as the selection bias and in the inter-chunk softmax).

Offload.  Past the reference's thresholds (hidden size >= 4096 and more than 128K tokens,
utils/hils_cache_utils.py:4-5,19-23) the reference moves K and V to pinned host memory and copies the
whole cache back to the GPU on every update (:44-60).  Here K and V then LIVE in pinned host memory
and are read in place: a decode step touches only the pooled chunk keys (which stay on the GPU), the
top-k selected chunks and the local window, so the kernels fetch exactly those rows over the host
link instead of the whole cache.  ``update`` then returns pinned host views."""
import math

import torch

try:  # imported as part of the package ...
    from ..ops import _cabi
    from ..ops.chunk_attn_pool_tilelang import chunk_attn_pool, chunk_mean_pool
    from ..ops.hils_fwd_bwd_head import HiLS_block_M_head
    from ..ops.hils_glue import chunk_weights, decode_step, topk_chunk_weights
    from ..ops.topk_head_softmax import online_softmax_topk_head
except ImportError:  # ... or with the package directory itself on sys.path (`from utils... import`)
    from ops import _cabi
    from ops.chunk_attn_pool_tilelang import chunk_attn_pool, chunk_mean_pool
    from ops.hils_fwd_bwd_head import HiLS_block_M_head
    from ops.hils_glue import chunk_weights, decode_step, topk_chunk_weights
    from ops.topk_head_softmax import online_softmax_topk_head


_OFFLOAD_SEQ_THRESHOLD = 128 * 1024
_OFFLOAD_HIDDEN_DIM_THRESHOLD = 4096


def _attention_pooled(mu_q, k_chunks, num_kv_heads):
    """Prior queries mu_q (B,n,h_q,D) over the chunks k_chunks (B,n,S,H,D): attention-pooled keys
    (B,n,h_q,D) and entropy bias (B,n,h_q) fp32 (models/FlashHiLS/hils_attention.py:66-135; K stays
    at its own head count)."""
    assert k_chunks.shape[3] == num_kv_heads
    lk, lb = chunk_attn_pool(mu_q.contiguous(), k_chunks.contiguous())
    return lk, lb.float()


class HiLSDynamicLayer:
    """update() / get_seq_length() as in the reference's class; the buffers grow by doubling.
    ``offload``: None = by the reference's thresholds, True / False = forced.
    ``chunk_pooling``: the chunk keys are the chunk means (the layer's ``enable_chunk_pooling``); when
    ``update`` is also given the prior queries ``mu_q`` of the chunks it completes, the entropy bias of
    the attention pool is kept beside them (``enable_prior_query``).  With ``chunk_pooling=False`` the
    attention-pooled keys themselves are the chunk keys (one per query head)."""

    is_sliding = False

    def __init__(self, chunk_size=64, capacity=0, offload=None, chunk_pooling=True):
        self.chunk_size = int(chunk_size)
        self.capacity = int(capacity)
        self.seq_len = 0
        self.pooled_chunks = 0  # chunks whose pooled key is in the buffers
        self.keys = self.values = None
        self._lmk_hm = None     # (B, H or h_q, capacity / S, D): chunk keys, head-major
        self._prior_hm = None   # (B, H, capacity / S, G) fp32: prior bias, once mu_q has been seen
        self.chunk_pooling = bool(chunk_pooling)
        self.is_initialized = False
        self._offload_choice = offload
        self._offloading = False
        self._hidden_dim = 0

    # the reference's layouts, as views of the head-major buffers
    @property
    def lmk_k(self):
        """(B, chunks, heads, D) view of the chunk keys."""
        return None if self._lmk_hm is None else self._lmk_hm.permute(0, 2, 1, 3)

    @property
    def prior_b(self):
        """(B, chunks, h_q) view-copy of the prior bias (None before any ``mu_q``)."""
        if self._prior_hm is None:
            return None
        B, H, n, G = self._prior_hm.shape
        return self._prior_hm.permute(0, 2, 1, 3).reshape(B, n, H * G)

    def _should_offload(self, new_seq_len):
        if self._offload_choice is not None:
            return bool(self._offload_choice)
        return self._hidden_dim >= _OFFLOAD_HIDDEN_DIM_THRESHOLD and new_seq_len > _OFFLOAD_SEQ_THRESHOLD

    def _kv_buffer(self, shape):
        """K / V storage: device memory, or pinned host memory once the layer offloads."""
        if self._offloading:
            return torch.zeros(shape, dtype=self.dtype, device="cpu", pin_memory=True)
        return torch.zeros(shape, dtype=self.dtype, device=self.device)

    def _move_to_host(self):
        self._offloading = True
        for name in ("keys", "values"):
            old = getattr(self, name)
            new = self._kv_buffer(tuple(old.shape))
            new[:, : self.seq_len].copy_(old[:, : self.seq_len], non_blocking=True)
            setattr(self, name, new)
        torch.cuda.current_stream().synchronize()

    def lazy_initialization(self, key_states, value_states):
        B, T, H, D = key_states.shape
        S = self.chunk_size
        cap = max(self.capacity, T, S)
        cap = (cap + S - 1) // S * S
        self.capacity = cap
        self.dtype, self.device = key_states.dtype, key_states.device
        self._hidden_dim = H * D
        self._offloading = self._should_offload(T)
        self.keys = self._kv_buffer((B, cap, H, D))
        self.values = self._kv_buffer((B, cap, H, value_states.shape[-1]))
        self.is_initialized = True

    def _grow(self, need):
        S = self.chunk_size
        cap = self.capacity
        while cap < need:
            cap *= 2
        cap = (cap + S - 1) // S * S
        for name in ("keys", "values"):
            old = getattr(self, name)
            new = self._kv_buffer((old.shape[0], cap) + tuple(old.shape[2:]))
            new[:, : old.shape[1]] = old
            setattr(self, name, new)
        for name in ("_lmk_hm", "_prior_hm"):
            old = getattr(self, name)
            if old is not None:
                new = torch.zeros(tuple(old.shape[:2]) + (cap // S,) + tuple(old.shape[3:]), dtype=old.dtype,
                                  device=old.device)
                new[:, :, : old.shape[2]] = old
                setattr(self, name, new)
        self.capacity = cap

    def update(self, key_states, value_states, *args, mu_q=None, **kwargs):
        """Append (B, T, H, D) keys / values; pool the chunks they complete.  ``mu_q``
        (B, new_full_chunks, h_q, D): the prior queries of those chunks (attention-pooled prior).
        Returns views of the valid part of the cache (what the reference's update returns)."""
        if not self.is_initialized:
            self.lazy_initialization(key_states, value_states)
        T = key_states.shape[1]
        if not self._offloading and self._should_offload(self.seq_len + T):
            self._move_to_host()
        if self.seq_len + T > self.capacity:
            self._grow(self.seq_len + T)
        a, b = self.seq_len, self.seq_len + T
        self.keys[:, a:b].copy_(key_states, non_blocking=True)
        self.values[:, a:b].copy_(value_states, non_blocking=True)
        if self._offloading:  # the host copies are complete before anything reads the buffers
            torch.cuda.current_stream().synchronize()
        self.seq_len = b
        S = self.chunk_size
        full = b // S
        if full > self.pooled_chunks:
            c0 = self.pooled_chunks
            B, H, D = key_states.shape[0], key_states.shape[2], key_states.shape[3]
            src = self.keys[:, c0 * S: full * S]
            if self._offloading:  # the tokens of the chunks just completed: a small copy back
                src = src.to(self.device, non_blocking=True)
            src = src.contiguous()
            pooled = chunk_mean_pool(src, S) if (self.chunk_pooling or mu_q is None) else None
            if mu_q is not None:
                h_q = mu_q.shape[2]
                assert mu_q.shape == (B, full - c0, h_q, D) and h_q % H == 0, f"mu_q shape {tuple(mu_q.shape)}"
                lk, lb = _attention_pooled(mu_q, src.view(B, full - c0, S, H, D), H)
                if self._prior_hm is None:
                    assert c0 == 0, "the prior bias must be kept from the first chunk on"
                    self._prior_hm = torch.zeros((B, H, self.capacity // S, h_q // H), dtype=torch.float32,
                                                 device=self.device)
                self._prior_hm[:, :, c0:full] = lb.view(B, full - c0, H, h_q // H).permute(0, 2, 1, 3)
                if pooled is None:
                    pooled = lk  # one chunk key per query head
            else:
                assert self._prior_hm is None, "this cache keeps a prior bias: update() needs mu_q for new chunks"
            if self._lmk_hm is None:
                self._lmk_hm = torch.zeros((B, pooled.shape[2], self.capacity // S, D), dtype=self.dtype,
                                           device=self.device)
            self._lmk_hm[:, :, c0:full] = pooled.permute(0, 2, 1, 3)
            self.pooled_chunks = full
        return self.keys[:, :b], self.values[:, :b]

    def get_seq_length(self):
        return self.seq_len

    def get_mask_sizes(self, query_length):
        return self.seq_len + query_length, 0

    def get_max_cache_shape(self):
        return -1

    def hils_attend(self, q, lse_swa, topk, window_size, sm_scale=None, _debug=None):
        """The remote (HiLS) branch for the last ``q.shape[1]`` positions of the cache: chunk
        selection, inter-chunk softmax (with the prior bias when the cache keeps one) and sparse
        attention on the cache buffers in place.  q (B, Lq, h_q, D) bf16, lse_swa (B, Lq, h_q) of the
        local branch.  Returns (o_remote (B, Lq, h_q, Dv), weights (B, Lq, h_q, topk + 1), indices);
        the layer adds ``swa_o * weights[..., topk]`` to o_remote."""
        assert self.is_initialized and q.shape[1] <= self.seq_len and self._lmk_hm is not None
        S = self.chunk_size
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(q.shape[-1])
        H = self.keys.shape[2]
        q_offset = self.seq_len - q.shape[1]
        # one launch when the shape allows it (decode_step falls back to the two calls otherwise); the chunk
        # keys are per KV head or, kept from the attention pool, per query head
        o, w, idx, _ = decode_step(q, self._lmk_hm, self.keys, self.values, lse_swa, topk, S, window_size,
                                   q_offset=q_offset, sm_scale=sm_scale, prior_b=self._prior_hm,
                                   lmk_head_major=True, num_chunks=max(self.pooled_chunks, 1), _debug=_debug)
        return o, w, idx


class HiLSPagedLayer:
    """KV cache of one HiLS layer in pages of one chunk (64 tokens), the layout a paged serving
    backend keeps (the reference's SGLang backend requires page size = chunk size, README.md:262-264).

    ``k_pages`` / ``v_pages``: (num_pages, H, 64, D), the 64 tokens of a (page, head) contiguous;
    (with ``chunk_pooling=False`` and ``num_q_heads`` the chunk keys below carry h_q heads, one per query head)
    ``page_table``: (B, max_pages) int32, chunk c of sequence b -> page, -1 = not mapped.  The pooled
    key of every full chunk is kept twice: per page in ``lmk_pages`` (num_pages, H, D) (with
    ``prior_pages`` (num_pages, h_q) beside it), and per sequence, dense and head-major, in ``lmk_hm``
    (B, H, max_pages, D) / ``prior_hm`` (B, H, max_pages, G), which is what ``hils_attend`` streams (a
    row's keys are contiguous there; the reference keeps them per layer in ``_hils_prior_cache``,
    models/FlashHiLS/hils_attention.py:361-416).  The pooled key is the mean of the chunk's 64 keys, or,
    when ``update`` is given the chunks' prior queries ``mu_q``, the attention pool's entropy bias is
    kept too (and its pooled key replaces the mean unless ``chunk_pooling``).  All sequences of the batch
    have the same length (the kernels take one query offset, as the reference's do).  Pages come from a
    free list, so the page order of a sequence is arbitrary."""

    def __init__(self, num_pages, batch, max_pages_per_seq, num_kv_heads, head_dim, device,
                 num_q_heads=None, chunk_pooling=True, page_order=None, dtype=torch.bfloat16):
        self.S = 64
        self.B, self.H, self.D = int(batch), int(num_kv_heads), int(head_dim)
        self.num_pages, self.max_pages = int(num_pages), int(max_pages_per_seq)
        self.k_pages = torch.zeros((num_pages, self.H, self.S, self.D), dtype=dtype, device=device)
        self.v_pages = torch.zeros_like(self.k_pages)
        self.chunk_pooling = bool(chunk_pooling)
        # chunk keys per KV head (chunk means) or, kept from the attention pool, per query head
        self.h_lmk = self.H if (self.chunk_pooling or num_q_heads is None) else int(num_q_heads)
        self.lmk_pages = torch.zeros((num_pages, self.h_lmk, self.D), dtype=dtype, device=device)
        self.lmk_hm = torch.zeros((self.B, self.h_lmk, self.max_pages, self.D), dtype=dtype, device=device)
        self.prior_pages = self.prior_hm = None
        self.has_prior = False  # set once update() has been given prior queries
        if num_q_heads is not None:
            G = int(num_q_heads) // self.H
            self.prior_pages = torch.zeros((num_pages, int(num_q_heads)), dtype=torch.float32, device=device)
            self.prior_hm = torch.zeros((self.B, self.H, self.max_pages, G), dtype=torch.float32, device=device)
        self.page_table = torch.full((self.B, self.max_pages), -1, dtype=torch.int32, device=device)
        # pages are handed out from the end of this list
        order = list(range(num_pages - 1, -1, -1)) if page_order is None else [int(p) for p in reversed(page_order)]
        self.free_pages = order
        self.seq_len = 0
        self.pooled_chunks = 0

    @property
    def prior_b(self):
        """The entropy bias per page, (num_pages, h_q) fp32 (None without ``num_q_heads``)."""
        return self.prior_pages

    def get_seq_length(self):
        return self.seq_len

    def update(self, key_states, value_states, mu_q=None):
        """Append (B, T, H, D) keys / values.  ``mu_q`` (B, new_full_chunks, h_q, D): the prior queries
        of the chunks this call completes; with it the entropy bias of the attention pool is kept and
        used by ``hils_attend`` (and the attention-pooled keys are the chunk keys unless
        ``chunk_pooling``)."""
        B, T, H, D = key_states.shape
        assert (B, H, D) == (self.B, self.H, self.D)
        S, dev = self.S, self.k_pages.device
        a, b_end = self.seq_len, self.seq_len + T
        need = (b_end + S - 1) // S
        have = (a + S - 1) // S
        assert need <= self.max_pages, "the page table is too short for this sequence length"
        if need > have:
            n_new = (need - have) * B
            assert n_new <= len(self.free_pages), "out of pages"
            new = torch.tensor([self.free_pages.pop() for _ in range(n_new)], dtype=torch.int32,
                               device=dev).view(need - have, B).t()
            self.page_table[:, have:need] = new
        pos = torch.arange(a, b_end, device=dev)
        pages = self.page_table[:, pos // S].long()                      # (B, T)
        slots = (pos % S).view(1, T).expand(B, T)
        hh = torch.arange(H, device=dev).view(1, 1, H)
        self.k_pages[pages.unsqueeze(-1), hh, slots.unsqueeze(-1)] = key_states
        self.v_pages[pages.unsqueeze(-1), hh, slots.unsqueeze(-1)] = value_states
        self.seq_len = b_end
        full = b_end // S
        if full > self.pooled_chunks:
            c0 = self.pooled_chunks
            n = full - c0
            pg = self.page_table[:, c0:full].long().reshape(-1)          # (B * n) pages, batch-major
            kk = self.k_pages[pg]                                        # (B*n, H, 64, D), a copy
            pooled = None
            if self.chunk_pooling or mu_q is None:
                # every (page, head) is a 64-token sequence of its own for the pooling kernel
                pooled = chunk_mean_pool(kk.view(-1, S, 1, D), S).view(-1, H, D)
            if mu_q is not None:
                hq = mu_q.shape[2]
                G = hq // H
                assert mu_q.shape == (B, n, hq, D), f"mu_q shape {tuple(mu_q.shape)}"
                assert self.prior_pages is not None, "construct the layer with num_q_heads to keep a prior bias"
                assert c0 == 0 or self.has_prior, "the prior bias must be kept from the first chunk on"
                lk, lb = _attention_pooled(mu_q.reshape(-1, 1, hq, D), kk.permute(0, 2, 1, 3).unsqueeze(1), H)
                self.prior_pages[pg] = lb.reshape(-1, hq)
                self.prior_hm[:, :, c0:full] = lb.view(B, n, H, G).permute(0, 2, 1, 3)
                self.has_prior = True
                if pooled is None:
                    assert hq == self.h_lmk, "attention-pooled chunk keys are per query head"
                    pooled = lk.reshape(-1, hq, D)
            else:
                assert not self.has_prior, "this cache keeps a prior bias: update() needs mu_q for new chunks"
            assert pooled.shape[1] == self.h_lmk, (
                "a layer built without chunk pooling keeps the attention pool's keys: update() needs mu_q")
            pooled = pooled.to(self.lmk_pages.dtype)
            self.lmk_pages[pg] = pooled
            self.lmk_hm[:, :, c0:full] = pooled.view(B, n, self.h_lmk, D).permute(0, 2, 1, 3)
            self.pooled_chunks = full

    def gather_contiguous(self):
        """(B, seq_len, H, D) keys and values in token order (for the local branch, or checks)."""
        S = self.S
        n = (self.seq_len + S - 1) // S
        pg = self.page_table[:, :n].long()
        k = self.k_pages[pg].permute(0, 1, 3, 2, 4).reshape(self.B, n * S, self.H, self.D)[:, : self.seq_len]
        v = self.v_pages[pg].permute(0, 1, 3, 2, 4).reshape(self.B, n * S, self.H, self.D)[:, : self.seq_len]
        return k.contiguous(), v.contiguous()

    def hils_attend(self, q, lse_swa, topk, window_size, sm_scale=None, _debug=None, dense_keys=True):
        """The remote branch for the last ``q.shape[1]`` positions: selection, inter-chunk softmax (with
        the prior bias once ``update`` has been given prior queries) and sparse attention straight on
        the pages.  ``dense_keys``: stream the per-sequence head-major chunk keys (default) instead of
        the per-page ones.  Returns (o (B,Lq,h_q,D), weights (B,Lq,h_q,topk+1), indices (B,Lq,H,topk)
        as chunk numbers of the sequence)."""
        if dense_keys:
            return paged_hils_attend(q, self.k_pages, self.v_pages, None, self.page_table, lse_swa, self.seq_len,
                                     topk, window_size, sm_scale=sm_scale, _debug=_debug, lmk_dense=self.lmk_hm,
                                     prior_dense=self.prior_hm if self.has_prior else None)
        return paged_hils_attend(q, self.k_pages, self.v_pages, self.lmk_pages, self.page_table, lse_swa,
                                 self.seq_len, topk, window_size, sm_scale=sm_scale, _debug=_debug,
                                 prior_pages=self.prior_pages if self.has_prior else None)


def paged_hils_attend(q, k_pages, v_pages, lmk_pages, page_table, lse_swa, seq_len, topk, window_size,
                      sm_scale=None, _debug=None, prior_pages=None, lmk_dense=None, prior_dense=None):
    """Selection + inter-chunk softmax + sparse attention of the last ``q.shape[1]`` positions of a
    ``seq_len``-token sequence kept in pages (layouts: see ``HiLSPagedLayer``).  Chunk keys: per page
    (``lmk_pages`` (num_pages,H,D), prior bias ``prior_pages`` (num_pages,h_q)) or per sequence,
    head-major (``lmk_dense`` (B,H,cap,D), prior bias ``prior_dense`` (B,H,cap,G)); either may carry h_q
    heads in place of H (one chunk key per query head); the prior bias, when given, is the selection
    bias and the bias of the inter-chunk softmax (models/FlashHiLS/hils_attention.py:568-602)."""
    dense = lmk_dense is not None
    _cabi.require_gpu_bf16("paged_hils_attend", q, k_pages, v_pages, lmk_dense if dense else lmk_pages)
    B, Lq, HQ, D = q.shape
    num_pages, H, S, Dk = k_pages.shape
    assert S == 64 and Dk == D and v_pages.shape == k_pages.shape
    assert page_table.dtype == torch.int32 and page_table.shape[0] == B and page_table.is_contiguous()
    assert HQ % H == 0
    G = HQ // H
    max_pages = page_table.shape[1]
    N = seq_len // S  # chunks with a pooled key
    assert 0 < N <= max_pages
    cap = 0
    h_lmk = lmk_dense.shape[1] if dense else lmk_pages.shape[1]
    assert h_lmk in (H, HQ), f"the chunk keys carry {h_lmk} heads: neither the {H} KV heads nor the {HQ} query heads"
    per_qhead = int(h_lmk != H)
    if dense:
        cap = lmk_dense.shape[2]
        assert lmk_dense.shape == (B, h_lmk, cap, D) and lmk_dense.is_contiguous() and cap >= N
        bias = None
        if prior_dense is not None:
            assert prior_dense.shape == (B, H, cap, G) and prior_dense.dtype == torch.float32
            bias = prior_dense.contiguous()
        lmk_arg = lmk_dense
    else:
        assert lmk_pages.shape == (num_pages, h_lmk, D) and lmk_pages.is_contiguous()
        bias = None
        if prior_pages is not None:
            assert prior_pages.shape == (num_pages, HQ) and prior_pages.dtype == torch.float32
            bias = prior_pages.contiguous()
        lmk_arg = lmk_pages
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    dev = q.device
    lse = lse_swa.reshape(B, Lq, HQ).float().contiguous()
    indices = torch.empty((B, Lq, H, topk), dtype=torch.int32, device=dev)
    scores = torch.empty((B, Lq, HQ, topk), dtype=q.dtype, device=dev)
    weights = torch.empty((B, Lq, HQ, topk + 1), dtype=q.dtype, device=dev)
    lse_total = sel_logits = None
    if _debug is not None:
        lse_total = torch.empty((B, Lq, H, G), dtype=torch.float32, device=dev)
        sel_logits = torch.full((B, Lq, H, G, N), float("-inf"), dtype=torch.float32, device=dev)
    qc = q.contiguous()
    if _cabi.load().hils_decode_step_covers(B, Lq, N, HQ, H, D, int(topk), S, int(bias is not None)):
        # selection and attention of a row by one workgroup, one launch
        o = torch.empty((B, Lq, HQ, D), dtype=q.dtype, device=dev)
        _cabi.call("hils_decode_step_paged", _cabi.ptr(qc), _cabi.ptr(lmk_arg), _cabi.ptr(k_pages),
                   _cabi.ptr(v_pages), _cabi.ptr(page_table), _cabi.ptr(lse), _cabi.ptr(bias), _cabi.ptr(indices),
                   _cabi.ptr(scores), _cabi.ptr(weights), _cabi.ptr(o), _cabi.ptr(lse_total), _cabi.ptr(sel_logits),
                   B, Lq, N, HQ, H, D, int(topk), S, int(window_size), seq_len - Lq, max_pages, num_pages,
                   float(sm_scale), float(sm_scale), 1, int(dense), int(dense), cap, per_qhead)
        if _debug is not None:
            _debug.update(lse_total=lse_total, sel_logits=sel_logits, scores=scores)
        return o, weights, indices
    if dense:
        # shapes outside the one-launch kernel: selection and softmax on the reference's dense layout,
        # attention on the pages
        lmk_tm = lmk_dense[:, :, :N].permute(0, 2, 1, 3).contiguous()
        pb = None if bias is None else bias[:, :, :N].permute(0, 2, 1, 3).reshape(B, N, HQ).contiguous()
        indices, scores, weights = topk_chunk_weights(qc, lmk_tm, lse, topk, S, window_size,
                                                      q_offset=seq_len - Lq, sm_scale=sm_scale, prior_b=pb,
                                                      num_kv_heads=H)
        if _debug is not None:
            _debug.update(scores=scores)
    else:
        _cabi.call("hils_topk_fwd_weights_paged", _cabi.ptr(qc), _cabi.ptr(lmk_pages), _cabi.ptr(page_table),
                   _cabi.ptr(lse), _cabi.ptr(bias), _cabi.ptr(indices), _cabi.ptr(scores), _cabi.ptr(weights),
                   _cabi.ptr(lse_total), _cabi.ptr(sel_logits), B, Lq, N, H, G, D, int(topk), S, int(window_size),
                   seq_len - Lq, max_pages, num_pages, float(sm_scale), per_qhead)
        if _debug is not None:
            _debug.update(lse_total=lse_total, sel_logits=sel_logits, scores=scores)
    o = torch.empty((B, Lq, HQ, D), dtype=q.dtype, device=dev)
    n_ws = _cabi.load().hils_sparse_attn_decode_paged_workspace(B, Lq, HQ, H, D, int(topk))
    ws = torch.empty(n_ws, dtype=torch.uint8, device=dev) if n_ws else None
    _cabi.call("hils_sparse_attn_decode_paged", _cabi.ptr(qc), _cabi.ptr(k_pages), _cabi.ptr(v_pages),
               _cabi.ptr(page_table), _cabi.ptr(weights), _cabi.ptr(indices), _cabi.ptr(o), _cabi.ptr(ws), _cabi.nbytes(ws),
               B, Lq, HQ, H, D, int(topk), topk + 1, max_pages, num_pages, float(sm_scale), 1)
    return o, weights, indices
