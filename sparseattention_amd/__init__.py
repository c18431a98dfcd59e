"""MI355X-native block-sparse attention forward.

Same Python surface as tomatillos/sparseattention for its one hot path:

* :func:`sparse_attention` (reference: ``sparseattention/sparse_attn_kernel.py:149``)
* :func:`sparse_attention_decode`: the same function for Sq <= 32 with a split-KV launch (the reference names
  decode kernels as future work, ``README.md:65``)
* :func:`compute_mask_kernel`, :func:`compute_mask_slow`, :class:`MaskMetadata`
  (reference: ``sparseattention/mask_utils.py:85``, ``:14``, ``:6``)
* :func:`compute_mask_terms`: the same metadata for masks given by a formula (:class:`MaskTerm`), without the
  Sq x Sk tensor (the reference names algebraic masks as future work, ``README.md:63``)

The device work is done by hand-written gfx950 HIP kernels in ``libsparseattn_hip.so``
behind the C ABI of ``include/sparseattn.h``.
"""
from .mask_utils import (MaskMetadata, MaskTerm, block_term, causal_term, compute_mask_kernel, compute_mask_slow,
                         compute_mask_terms, materialize_mask_terms, select_block_sizes, select_tiling, Tiling,
                         with_list_stats)
from .sparse_attn_kernel import (BackwardMetadata, compute_backward_metadata, compute_backward_metadata_terms,
                                 merge_attention_parts, sparse_attention,
                                 sparse_attention_backward, sparse_attention_decode, sparse_attention_kv_split,
                                 sparse_attention_tiled, sparse_attention_trainable)

__all__ = ["MaskMetadata", "compute_mask_kernel", "compute_mask_slow", "select_block_sizes", "sparse_attention",
           "sparse_attention_decode", "sparse_attention_backward", "sparse_attention_trainable", "BackwardMetadata",
           "compute_backward_metadata", "merge_attention_parts", "sparse_attention_kv_split", "MaskTerm", "causal_term",
           "block_term", "compute_mask_terms", "materialize_mask_terms", "compute_backward_metadata_terms", "select_tiling",
           "Tiling", "sparse_attention_tiled", "with_list_stats"]
