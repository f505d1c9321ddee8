"""MI355X-native SpargeAttn hot path: same operator API as ``spas_sage_attn`` (thu-ml/SpargeAttn)."""
from .core import (spas_sage_attn_meansim_cuda, spas_sage2_attn_meansim_cuda, block_sparse_sage2_attn_cuda,
                   spas_sage_attn_meansim_topk_cuda, spas_sage2_attn_meansim_topk_cuda)

# the five names spas_sage_attn/__init__.py:1-7 exports
__all__ = ["spas_sage_attn_meansim_cuda", "spas_sage2_attn_meansim_cuda", "block_sparse_sage2_attn_cuda",
           "spas_sage_attn_meansim_topk_cuda", "spas_sage2_attn_meansim_topk_cuda"]
