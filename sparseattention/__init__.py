"""The reference's import paths over the MI355X implementation.

The reference's callers import ``sparseattention.sparse_attn_kernel.sparse_attention`` and
``sparseattention.mask_utils.compute_mask_kernel`` (sparseattention/test_attn.py:11-12); its ``__init__.py`` is
empty.  The modules of this package hold the objects of ``sparseattention_amd`` under those names, so code written
against the reference runs unedited once this repository's root is on ``sys.path`` in its place.
"""
