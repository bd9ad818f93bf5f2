"""fast_memory_amd: MI355X (gfx950) implementation of the indexed-memory
attention path of notbadai/fast_memory behind the reference's Python API.

All compute runs in hand-written HIP kernels reached through the C ABI of
``libfastmem.so`` (``include/fastmem.h``); PyTorch supplies device memory and
streams.  There is no CPU path.
"""
from .hash_attention import attention_hash, attention_hash_varlen, attention_hash_varlen_backward  # noqa: F401
from .memory import (Memory, MemoryBatch, calc_ref_centroids, compute_centroids, fit_projection, init_centroids, kmeans_spherical, learn_emb_proj,  # noqa: F401
                     merge, ring_attention_masked_backward, ring_attention_masked_forward, update_out_and_lse)

from .autograd import attention_hash_varlen_op, local_attention_backward, ring_cross_attention_approx  # noqa: F401,E402

__all__ = ["attention_hash_varlen_op", "local_attention_backward", "ring_cross_attention_approx", "attention_hash", "attention_hash_varlen", "attention_hash_varlen_backward", "Memory", "MemoryBatch", "calc_ref_centroids", "compute_centroids", "fit_projection",
           "init_centroids", "kmeans_spherical", "learn_emb_proj", "merge", "ring_attention_masked_backward", "ring_attention_masked_forward",
           "update_out_and_lse"]
