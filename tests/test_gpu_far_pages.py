"""GPU: every kernel of the path on pages that lie more than 2^32 bytes into a head's plane.

A pool of 200 000 pages x 128 slots x 128 bf16 is 6.5 GB per cached head, so the pages at its top are past the
reach of 32-bit byte offsets (and the second head's plane starts past it altogether).  The same steps run on a
64-page pool with the same pages in the same order; the large pool's top 64 pages must then hold the same bits
as the small pool, everything below them must be untouched, and every result must be identical: the two runs
differ in nothing but the page numbers.
"""

import math

import pytest
import torch

from falcon_perception_amd import ops
from tests.gpu_cases import DEV, randn

pytestmark = pytest.mark.gpu

P, D, HC, G = 128, 128, 2, 2
SMALL, LARGE = 64, 200_000
SHIFT = LARGE - SMALL  # page p of the small pool is page p + SHIFT of the large one
LENS = [300, 1000, 77]
DTYPE = torch.bfloat16


def tables(gen):
    """One page-table row per sequence over shuffled pages of the small pool, and the same rows moved up."""
    perm = (torch.randperm(SMALL - 1, generator=gen) + 1).tolist()
    small = torch.zeros((len(LENS) + 1, SMALL), dtype=torch.int64)
    large = torch.zeros((len(LENS) + 1, LARGE), dtype=torch.int64)
    for b, L in enumerate(LENS, start=1):
        for blk in range(-(-(L + 1) // P)):
            page = perm.pop()
            small[b, blk] = page
            large[b, blk] = page + SHIFT
    return small.to(DEV), large.to(DEV)


def pools(n_pages, H):
    return (torch.zeros((H, n_pages * P, D), dtype=DTYPE, device=DEV),
            torch.zeros((H, n_pages * P, D), dtype=DTYPE, device=DEV))


def same_pool(small, large):
    lo = SHIFT * P
    assert (large.shape[1] - lo) == small.shape[1] and lo * D * 2 > 2**32
    assert torch.equal(large[:, lo:].view(torch.int16), small.view(torch.int16))
    assert not large[:, :lo].view(torch.int16).any()


@pytest.mark.bigmem
def test_every_kernel_on_pages_beyond_4_gib():
    free, _ = torch.cuda.mem_get_info()
    assert free > 60e9, f"only {free / 1e9:.0f} GB of HBM free: this case holds about 30 GB"
    gen = torch.Generator().manual_seed(77)
    pt_s, pt_l = tables(gen)
    pk_s, pv_s = pools(SMALL, HC)
    pk_l, pv_l = pools(LARGE, HC)
    T = sum(LENS)
    bidx = torch.cat([torch.full((L,), b, dtype=torch.int64) for b, L in enumerate(LENS, start=1)])[None].to(DEV)
    pos = torch.cat([torch.arange(L, dtype=torch.int64) for L in LENS])[None].to(DEV)
    k = randn(gen, (1, HC, T, D), DTYPE).to(DEV)
    v = randn(gen, (1, HC, T, D), DTYPE).to(DEV)

    # packed prefill append
    for pk, pv, pt in ((pk_s, pv_s, pt_s), (pk_l, pv_l, pt_l)):
        ops.kv_append(pk, pv, k, v, pt, bidx, pos, P, clamp_negative=False, packed=True)
    same_pool(pk_s, pk_l)
    same_pool(pv_s, pv_l)

    # page gather
    slots = torch.arange(1, len(LENS) + 1, dtype=torch.int64, device=DEV)
    lens = torch.tensor(LENS, dtype=torch.int64, device=DEV)
    g_s = ops.kv_gather(pk_s, pt_s, slots, lens, P, max(LENS))
    g_l = ops.kv_gather(pk_l, pt_l, slots, lens, P, max(LENS))
    assert torch.equal(g_s.view(torch.int16), g_l.view(torch.int16)) and g_s.any()
    off = 0
    for i, L in enumerate(LENS):
        assert torch.equal(g_l[i, :, :L].view(torch.int16), k[0, :, off:off + L].view(torch.int16))
        off += L

    # chunked prefill attention over the pages: every row sees its causal prefix
    q = randn(gen, (1, HC * G, T, D), DTYPE).to(DEV)
    lim = (pos.view(-1) + 1).to(torch.int32)
    o_s, l_s = ops.paged_prefill(q, pk_s, pv_s, pt_s, bidx.view(-1), lim, P)
    o_l, l_l = ops.paged_prefill(q, pk_l, pv_l, pt_l, bidx.view(-1), lim, P)
    assert torch.equal(o_s.view(torch.int16), o_l.view(torch.int16)) and torch.equal(l_s, l_l) and o_s.any()

    # decode step with the append fused, split-K and the single-split direct store
    B = len(LENS)
    q1 = randn(gen, (B, HC * G, 1, D), DTYPE).to(DEV)
    k1, v1 = randn(gen, (B, HC, 1, D), DTYPE).to(DEV), randn(gen, (B, HC, 1, D), DTYPE).to(DEV)
    pos1 = torch.tensor(LENS, dtype=torch.int32, device=DEV)
    for split in (128, 2048):
        d_s = ops.paged_decode(q1, pk_s, pv_s, pt_s, slots, pos1, P, 1024, split_tokens=split, k_new=k1, v_new=v1)
        d_l = ops.paged_decode(q1, pk_l, pv_l, pt_l, slots, pos1, P, 1024, split_tokens=split, k_new=k1, v_new=v1)
        assert torch.equal(d_s[0].view(torch.int16), d_l[0].view(torch.int16)) and torch.equal(d_s[1], d_l[1])
        assert d_s[0].any()
    same_pool(pk_s, pk_l)
    same_pool(pv_s, pv_l)

    # the separate decode append (clamped), one more token per sequence
    pos2 = (pos1 + 1).view(B, 1)
    for pk, pv, pt in ((pk_s, pv_s, pt_s), (pk_l, pv_l, pt_l)):
        ops.kv_append(pk, pv, k1, v1, pt, slots, pos2, P, clamp_negative=True)
    same_pool(pk_s, pk_l)

    # QK norm + rotary + append in one launch, into emptied pools with one cached head per query head
    del pk_s, pv_s, pk_l, pv_l
    Hq = HC * G
    pk_s, pv_s = pools(SMALL, Hq)
    pk_l, pv_l = pools(LARGE, Hq)
    xq = randn(gen, (1, T, Hq, D), DTYPE).to(DEV)
    xk, xv = randn(gen, (1, T, HC, D), DTYPE).to(DEV), randn(gen, (1, T, HC, D), DTYPE).to(DEV)
    ang = torch.rand(1, T, D // 4, generator=gen) * 2 * math.pi
    f1 = torch.polar(torch.ones_like(ang), ang).to(DEV)
    ang2 = torch.randn(1, T, Hq, D // 4, generator=gen)
    f2 = torch.polar(torch.ones_like(ang2), ang2).to(DEV)
    r_s = ops.qkv_norm_rope_append(xq, xk, xv, f1, f2, pk_s, pv_s, pt_s, bidx.view(-1), pos.view(-1), P, clamp_negative=False)
    r_l = ops.qkv_norm_rope_append(xq, xk, xv, f1, f2, pk_l, pv_l, pt_l, bidx.view(-1), pos.view(-1), P, clamp_negative=False)
    assert torch.equal(r_s.view(torch.int16), r_l.view(torch.int16))
    same_pool(pk_s, pk_l)
    same_pool(pv_s, pv_l)
    assert pk_s.any() and pv_s.any()
