"""``sparseattention.mask_utils`` of the reference (mask_utils.py:6-11, :14-44, :85-107): the same names, bound to the
objects of :mod:`sparseattention_amd.mask_utils`."""
from sparseattention_amd.mask_utils import *  # noqa: F401,F403
from sparseattention_amd.mask_utils import (MaskMetadata, MaskTerm, block_term, causal_term,  # noqa: F401
                                            compute_mask_kernel, compute_mask_slow, compute_mask_terms,
                                            materialize_mask_terms, select_block_sizes)
