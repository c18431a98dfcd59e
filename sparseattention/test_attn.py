"""``python -m sparseattention.test_attn``: the reference's sweep (test_attn.py:79-149) under its own module path,
run by :mod:`sparseattention_amd.test_attn`."""
from sparseattention_amd.test_attn import do_bench, main, plot, random_blocked_mask, sweep, test_attn  # noqa: F401

if __name__ == "__main__":
    main()
