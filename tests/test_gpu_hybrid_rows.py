"""GPU parity: per-row key limits of the hybrid mask equal the oracle's dense mask rows."""

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV
from tests.test_oracle_masks import EOI, IMG, LAYOUTS, SOI, TXT, packed_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("layout", LAYOUTS)
def test_row_limits_on_engine_layouts(layout):
    ids, bidx, pos, spans = packed_case(layout)
    got = ops.hybrid_row_limits(torch.from_numpy(ids)[None].to(DEV), SOI, EOI).cpu().numpy()
    lo, hi = O.row_windows(bidx[None], ids[None], SOI, EOI)
    assert got.dtype == np.int32 and np.array_equal(got, hi)


@pytest.mark.parametrize("L", [1, 7, 1024, 1025, 5000, 65536])
def test_row_limits_on_random_delimiters(L):
    rng = np.random.default_rng(L)
    ids = rng.choice([SOI, EOI, IMG, TXT], size=L, p=[0.02, 0.02, 0.6, 0.36])
    got = ops.hybrid_row_limits(torch.from_numpy(ids).to(DEV), SOI, EOI).cpu().numpy()
    img, idx = O.image_prefix_tables(ids, SOI, EOI)
    # end of the run of equal (img, idx) that contains q, computed with numpy on the whole row
    key = np.where(img, idx, -1 - np.arange(L))  # non-image rows are runs of length one
    change = np.flatnonzero(np.diff(key) != 0) + 1
    ends = np.append(change, L)
    run_end = ends[np.searchsorted(ends, np.arange(L), side="right")]
    exp = np.where(img, run_end, np.arange(L) + 1)
    assert np.array_equal(got, exp)
    if L <= 5000:
        lo, hi = O.row_windows(np.ones((1, L), dtype=np.int64), ids[None], SOI, EOI)
        assert np.array_equal(got, hi)
