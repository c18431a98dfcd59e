"""``sparseattention.sparse_attn_kernel`` of the reference (sparse_attn_kernel.py:149-185): the same name, bound to
the objects of :mod:`sparseattention_amd.sparse_attn_kernel`."""
from sparseattention_amd.sparse_attn_kernel import *  # noqa: F401,F403
from sparseattention_amd.sparse_attn_kernel import (BackwardMetadata, compute_backward_metadata,  # noqa: F401
                                                    compute_backward_metadata_terms, kernel_tiles,
                                                    merge_attention_parts, sparse_attention,
                                                    sparse_attention_backward, sparse_attention_decode,
                                                    sparse_attention_kv_split, sparse_attention_trainable,
                                                    validate_metadata)
