"""The torch-CPU port that bench.py times as the CPU baseline computes what the oracle computes."""

import numpy as np
import torch

from oracle import cpu_path
from oracle import paged_kv_oracle as O


def test_cpu_port_matches_the_oracle():
    rng = np.random.default_rng(0)
    P, n_pages, Hc, G, D = 8, 24, 2, 2, 16
    a = O.PagedAllocator(n_pages, P, 5)
    a.free_pages = rng.permutation(np.arange(1, n_pages)).tolist()
    lens, slots = [13, 40, 8], []
    pool = np.zeros((1, 2, 1, Hc, n_pages * P, D), dtype=np.float32)
    for L in lens:
        b = a.allocate()
        a.reserve(b, L + 1)
        k = rng.standard_normal((1, Hc, L, D)).astype(np.float32)
        v = rng.standard_normal((1, Hc, L, D)).astype(np.float32)
        O.append_prefill(pool, 0, k, v, a.page_table, np.full((1, L), b), np.arange(L)[None], P)
        slots.append(b)
    k1 = rng.standard_normal((3, Hc, 1, D)).astype(np.float32)
    v1 = rng.standard_normal((3, Hc, 1, D)).astype(np.float32)
    q = rng.standard_normal((3, Hc * G, 1, D)).astype(np.float32)
    tpool = torch.from_numpy(pool.copy())
    out, lse = cpu_path.decode_step_cpu(tpool, 0, torch.from_numpy(a.page_table), torch.from_numpy(a.physical_to_logical),
                                        torch.tensor(slots), torch.tensor(lens), torch.from_numpy(k1),
                                        torch.from_numpy(v1), torch.from_numpy(q), P,
                                        logical_kv_indices=torch.zeros((3, 1, 1, 4), dtype=torch.int32))
    O.append_decode(pool, 0, k1, v1, a.page_table, np.array(slots), np.array(lens)[:, None], P)
    assert np.array_equal(tpool.numpy(), pool)
    eo, el = O.decode_attention(q, pool[0, 0, 0], pool[0, 1, 0], a.page_table, slots, lens, P)
    np.testing.assert_allclose(out.numpy(), eo, atol=1e-5, rtol=1e-5)
    np.testing.assert_allclose(lse.numpy(), el, atol=1e-5, rtol=1e-5)
