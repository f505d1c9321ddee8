"""MI355X-native SpargeAttn hot path: same operator API as ``spas_sage_attn`` (thu-ml/SpargeAttn)."""
from .core import (spas_sage2_attn_meansim_cuda, spas_sage2_attn_meansim_topk_cuda,
                   block_sparse_sage2_attn_cuda)

__all__ = ["spas_sage2_attn_meansim_cuda", "spas_sage2_attn_meansim_topk_cuda", "block_sparse_sage2_attn_cuda"]
