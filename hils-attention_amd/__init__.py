"""MI355X-native HiLS-Attention operator stack (hand-written gfx950 HIP kernels behind a C ABI).

The directory name carries a hyphen, so load it by path (see ``load_package`` in the
repository's ``__graft_entry__.py``) or put this directory on ``sys.path`` and import the
``ops`` sub-package under the reference's own module names, e.g.
``from ops.hils_fwd_bwd_head import HiLS_block_M_head``.
"""
from .ops.chunk_attn_pool_tilelang import (  # noqa: F401
    chunk_attn_pool, chunk_attn_pool_tilelang, chunk_attn_pool_tilelang_shared_k, chunk_mean_pool)
from .ops.topk_head_softmax import online_softmax_topk_head  # noqa: F401
from .ops.hils_fwd_bwd_head import HiLS_block_M_head  # noqa: F401
from .ops.hsa_triton import HSA  # noqa: F401
from .ops.exact_chunk_log_z_tilelang import exact_chunk_log_z_tl  # noqa: F401
from .ops.hils_glue import chunk_weights, decode_step, head_major_chunk_keys, topk_chunk_weights  # noqa: F401
from .ops.flex_attn_tilelang import flex_attn_tl, flex_attn_tl_two_phase  # noqa: F401
from .ops.hils_fwd_bwd_head import prepare_kv_workspace  # noqa: F401
from .utils.hils_cache_utils import HiLSDynamicLayer, HiLSPagedLayer, paged_hils_attend  # noqa: F401
from .ops.rope_tilelang_fp32 import rope_rotary_pos_emb, single_tensor_rope_autograd  # noqa: F401
from .ops.norm_rope_pool import norm_rope_pool  # noqa: F401
