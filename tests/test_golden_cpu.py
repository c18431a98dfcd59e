"""The C oracle against the committed known-answer files."""
import numpy as np
import pytest

import golden_io
import oracle
from helpers import assert_metadata_equal
from types import SimpleNamespace


@pytest.mark.parametrize("name", golden_io.names())
def test_oracle_matches_golden(name):
    g = golden_io.load(name)
    m4 = np.broadcast_to(g.mask[None, None], (g.B, g.H, g.S, g.S))
    meta = oracle.classify(m4, g.BQ, g.BK)
    plane = SimpleNamespace(**{f: getattr(meta, f)[0, 0] for f in ("unmasked_kv_ids", "unmasked_lens", "masked_kv_ids", "masked_lens")})
    assert_metadata_equal(plane, g.meta, name)
    q, k, v = (t.float().numpy() for t in (g.q, g.k, g.v))
    out = oracle.forward(q, k, v, m4, g.BQ, g.BK, meta=meta, p_round=0)
    assert np.abs(out - g.out).max() <= 1e-5
    out_bf16 = oracle.forward(q, k, v, m4, g.BQ, g.BK, meta=meta, p_round=1)
    assert np.abs(out_bf16 - g.out).max() <= 2e-2


def test_golden_files_exist():
    assert len(golden_io.names()) >= 4
