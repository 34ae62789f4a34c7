"""GPU parity: MFMA chunked-prefill attention over the paged cache under the hybrid mask,
against the float64 oracle.  Tolerance (north star): 2e-2 absolute / 1e-2 relative in bf16."""

import numpy as np
import pytest
import torch
from torch.nn.attention.flex_attention import AuxRequest

from falcon_perception_amd import attention as A
from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, f64, randn
from tests.test_oracle_masks import EOI, IMG, PAD, SOI, TXT, packed_case

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: (2e-2, 1e-2), torch.float16: (4e-3, 4e-3), torch.float32: (2e-5, 2e-5)}


# The bounded-score path multiplies Q by scale * log2(e) and rounds it to bf16 once more: a score, and with it
# the lse of a row that sees few keys, moves by up to |q||k| 2^-9 / sqrt(3 D) ~ 1e-3 per standard deviation.
BOUNDED_LSE_ATOL = 5e-3


def assert_close(out, lse, eo, el, dtype, rows=None, lse_atol=None):
    atol, rtol = TOL[dtype]
    go, gl = f64(out), f64(lse)
    if rows is not None:
        go, gl, eo, el = go[:, :, rows], gl[:, :, rows], eo[:, :, rows], el[:, :, rows]
    np.testing.assert_allclose(go, eo, atol=atol, rtol=rtol)
    np.testing.assert_allclose(gl, el, atol=lse_atol or max(atol * 0.1, 1e-4), rtol=rtol)


def prefill_through_api(st, ids, bidx, pos, Hq, dtype, pad_to):
    """insert_kv + compiled_flex_attn_prefill exactly as model.py:150-162 calls them."""
    cache = st.cache
    L = len(ids)
    t_ids = torch.from_numpy(ids)[None].to(DEV)
    t_b = torch.from_numpy(bidx)[None].to(DEV)
    t_p = torch.from_numpy(pos)[None].to(DEV)
    mask = cache.create_prefill_blockmask(t_b, t_ids, SOI, EOI)
    k = randn(st.gen, (1, st.Hc, L, st.D), dtype)
    v = randn(st.gen, (1, st.Hc, L, st.D), dtype)
    q = randn(st.gen, (1, Hq, L, st.D), dtype)
    K, V = cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=t_p, batch_idx=t_b)
    out, aux = A.compiled_flex_attn_prefill(q.to(DEV), K, V, block_mask=mask, return_aux=AuxRequest(lse=True),
                                            kernel_options={"FORCE_USE_FLEX_ATTENTION": True})
    return q, k, v, out, aux.lse


def layout_for(sizes):
    """One sequence per entry: (slot, text before, image tokens, text after)."""
    return [(slot, ([("t", a)] if a else []) + ([("i", n)] if n else []) + ([("t", b)] if b else []))
            for slot, a, n, b in sizes]


def repack(layout, pad_to):
    ids, bidx, pos = [], [], []
    for slot, segs in layout:
        start = len(ids)
        for kind, n in segs:
            ids += [TXT] * n if kind == "t" else [SOI] + [IMG + 1] * 4 + [IMG] * n + [EOI]
        L = len(ids) - start
        bidx += [slot] * L
        pos += list(range(L))
        gap = (-L) % pad_to
        ids += [PAD] * gap
        bidx += [0] * gap
        pos += [0] * gap
    return np.array(ids), np.array(bidx), np.array(pos)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("D,G", [(128, 1), (128, 2), (64, 4)])
def test_whole_sequence_prefill_matches_the_reference_semantics(dtype, D, G):
    """The reference's own prefill (packed sequences, each padded to 128): attention over the packed
    fresh K/V under image-prefix OR document-causal (paged_attention.py:343-393)."""
    Hc = 2
    layout = layout_for([(1, 5, 150, 40), (2, 0, 60, 200), (3, 131, 0, 0)])
    ids, bidx, pos = repack(layout, 128)
    st = PagedState(1, n_pages=64, page_size=64, max_batch=6, Hc=Hc, D=D, dtype=dtype)
    for slot in (1, 2, 3):
        st.add_sequence(int((bidx == slot).sum()))
    q, k, v, out, lse = prefill_through_api(st, ids, bidx, pos, Hc * G, dtype, 128)
    eo, el = O.prefill_attention_packed(f64(q), f64(k), f64(v), bidx[None], ids[None], SOI, EOI)
    real = np.flatnonzero(bidx != 0)
    assert_close(out, lse, eo, el, dtype, rows=real)
    pad = np.flatnonzero(bidx == 0)
    assert not f64(out)[:, :, pad].any() and np.isneginf(f64(lse)[:, :, pad]).all()


def test_unaligned_packing_and_small_pages():
    """Sequences packed back to back without padding (several sequences per 128-row tile), page size 16."""
    dtype = torch.bfloat16
    layout = layout_for([(1, 3, 20, 30), (2, 10, 0, 0), (3, 0, 40, 9), (4, 77, 0, 0), (5, 1, 0, 0)])
    ids, bidx, pos = repack(layout, 1)
    st = PagedState(2, n_pages=40, page_size=16, max_batch=8, Hc=2, D=128, dtype=dtype)
    for slot in (1, 2, 3, 4, 5):
        st.add_sequence(int((bidx == slot).sum()))
    q, k, v, out, lse = prefill_through_api(st, ids, bidx, pos, 4, dtype, 1)
    eo, el = O.prefill_attention_packed(f64(q), f64(k), f64(v), bidx[None], ids[None], SOI, EOI)
    assert_close(out, lse, eo, el, dtype)


@pytest.mark.parametrize("prefix,chunk", [(300, 100), (128, 128), (1000, 37), (0, 200)])
def test_chunk_over_a_paged_prefix(prefix, chunk):
    """Chunked prefill: the prefix (image span + text) is already in pages, the chunk's rows attend
    over prefix + chunk; equals the chunk's rows of the whole-sequence result."""
    dtype = torch.bfloat16
    Hc, G, D, P = 2, 2, 128, 64
    total = prefix + chunk
    n_img = max(0, min(prefix - 10, 200))
    ids = np.array(([TXT] * 2 + [SOI] + [IMG] * n_img + [EOI] if n_img else []) + [TXT] * total)[:total]
    st = PagedState(3, n_pages=40, page_size=P, max_batch=4, Hc=Hc, D=D, dtype=dtype)
    b = st.add_sequence(total)
    bidx = np.full(total, b)
    pos = np.arange(total)
    k = randn(st.gen, (1, Hc, total, D), dtype)
    v = randn(st.gen, (1, Hc, total, D), dtype)
    q = randn(st.gen, (1, Hc * G, total, D), dtype)
    cache = st.cache
    dev = lambda a: torch.from_numpy(a)[None].to(DEV)
    if prefix:
        cache.insert_kv(0, k[:, :, :prefix].to(DEV), v[:, :, :prefix].to(DEV), input_pos=dev(pos[:prefix]),
                        batch_idx=dev(bidx[:prefix]))
    # the chunk step: mask from the chunk's own tokens, positions continue after the prefix
    mask = cache.create_prefill_blockmask(dev(bidx[prefix:]), dev(ids[prefix:]), SOI, EOI)
    K, V = cache.insert_kv(0, k[:, :, prefix:].to(DEV), v[:, :, prefix:].to(DEV), input_pos=dev(pos[prefix:]),
                           batch_idx=dev(bidx[prefix:]))
    out, aux = A.compiled_flex_attn_prefill(q[:, :, prefix:].to(DEV), K, V, block_mask=mask,
                                            return_aux=AuxRequest(lse=True))
    eo, el = O.prefill_attention_packed(f64(q), f64(k), f64(v), bidx[None], ids[None], SOI, EOI)
    assert_close(out, aux.lse, eo[:, :, prefix:], el[:, :, prefix:], dtype)


def test_row_limits_direct_and_empty_rows():
    """ops.paged_prefill with explicit limits: limit 0 gives out 0 / lse -inf; limits beyond the row's
    own position give bidirectional attention."""
    dtype = torch.bfloat16
    st = PagedState(4, n_pages=16, page_size=32, max_batch=4, Hc=1, D=64, dtype=dtype)
    b = st.add_sequence(150)
    k, v, bt, pt, _, _ = st.prefill_random()
    q = randn(st.gen, (1, 2, 150, 64), dtype)
    lim = torch.randint(0, 151, (150,), generator=st.gen, dtype=torch.int32)
    lim[:5] = 0
    bidx = torch.full((150,), b, dtype=torch.int64)
    pk, pv = st.pool_planes()
    out, lse = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx.to(DEV), lim.to(DEV), st.P)
    eo, el = O.prefill_attention_paged(f64(q), f64(pk), f64(pv), st.mirror.page_table, bidx.numpy(),
                                       np.arange(150), lim.numpy(), st.P)
    assert_close(out, lse, eo, el, dtype)
    assert not f64(out)[:, :, :5].any() and np.isneginf(f64(lse)[:, :, :5]).all()


def test_cfg3_chunked_prefill_shape():
    """BASELINE configs[2]: 8 sequences, image prefix U[256,4096] already paged, 512-token text chunk each,
    16 q / 8 kv heads, D 128, page 128.  Checked on the first and last sequences (the oracle is O(L^2))."""
    import bench

    case = bench.make_prefill_case("cfg3", device=DEV)
    case.use_bound = False  # the online softmax with its running maximum
    out, lse = case.run()
    pk, pv = case.pool_k.float().cpu().numpy(), case.pool_v.float().cpu().numpy()
    bidx = case.batch_idx.cpu().numpy().reshape(-1)
    lim = case.row_limit.cpu().numpy()
    for s in (0, len(case.slots) - 1):
        rows = np.flatnonzero(bidx == case.slots[s])[::7]  # every 7th row of the chunk
        eo, el = O.prefill_attention_paged(f64(case.q[:, :, rows]), pk, pv, case.page_table.cpu().numpy(),
                                           bidx[rows], None, lim[rows], case.page_size)
        assert_close(out[:, :, rows], lse[:, :, rows], eo, el, torch.bfloat16)


def test_fp32_rows_over_a_long_context_with_small_pages():
    """fp32 (the reference's default dtype) on its own MFMA kernel: page size 16 is smaller than the
    kernel's 32-key tile, so every tile is staged row by row; limits around 8192 and a padding row."""
    dtype, P, D = torch.float32, 16, 64
    st = PagedState(9, n_pages=640, page_size=P, max_batch=3, Hc=1, D=D, dtype=dtype)
    b = st.add_sequence(9000)
    st.prefill_random()
    lims = [0, 1, 8191, 8192, 8193, 9000, 16 * 512 + 16 * 3 + 5]
    q = randn(st.gen, (1, 2, len(lims), D), dtype)
    bidx = torch.full((len(lims),), b, dtype=torch.int64)
    bidx[1] = 0  # a padding row: out 0, lse -inf whatever its limit
    lim = torch.tensor(lims, dtype=torch.int32)
    pk, pv = st.pool_planes()
    out, lse = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx.to(DEV), lim.to(DEV), P)
    eo, el = O.prefill_attention_paged(f64(q), f64(pk), f64(pv), st.mirror.page_table, bidx.numpy(),
                                       None, lim.numpy(), P)
    assert_close(out, lse, eo, el, dtype)
    assert not f64(out)[:, :, :2].any() and np.isneginf(f64(lse)[:, :, :2]).all()
    assert lse.shape == (1, 2, len(lims))


def test_a_run_longer_than_the_tile_slot_table():
    """The MFMA kernel looks up the first pool slot of up to 2048 tiles (131072 keys) of a run ahead of its
    tile loop; the tiles beyond, like the last tile of any run, are staged row by row.  Limits on both sides
    of that boundary, one of them ending inside a tile."""
    dtype, P, D = torch.bfloat16, 128, 64
    L = 2048 * 64 + 300
    st = PagedState(11, n_pages=L // P + 8, page_size=P, max_batch=3, Hc=1, D=D, dtype=dtype)
    b = st.add_sequence(L)
    st.prefill_random()
    lims = [2048 * 64 - 1, 2048 * 64, 2048 * 64 + 1, 2048 * 64 + 64, 2048 * 64 + 150, L]
    q = randn(st.gen, (1, 2, len(lims), D), dtype)
    bidx = torch.full((len(lims),), b, dtype=torch.int64)
    lim = torch.tensor(lims, dtype=torch.int32)
    pk, pv = st.pool_planes()
    out, lse = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx.to(DEV), lim.to(DEV), P)
    eo, el = O.prefill_attention_paged(f64(q), f64(pk), f64(pv), st.mirror.page_table, bidx.numpy(),
                                       None, lim.numpy(), P)
    assert_close(out, lse, eo, el, dtype)


@pytest.mark.parametrize("cut", [40, 101, 212])
def test_chunk_boundary_inside_the_image_span(cut):
    """A sequence of text + image block + text prefilled in two chunks whose boundary lies inside the
    image span (rows 12 .. 211, eoi at 212).  The first chunk cannot be served (its span rows would need
    keys that are not cached yet) and is refused; prefilled causally instead (K/V only matter), the second
    chunk declared with open_spans equals the rows of the whole-sequence result."""
    dtype = torch.bfloat16
    Hc, G, D, P = 2, 2, 128, 64
    ids = np.array([TXT] * 12 + [SOI] + [IMG + 1] * 4 + [IMG] * 195 + [EOI] + [TXT] * 60)
    total = len(ids)
    st = PagedState(21, n_pages=16, page_size=P, max_batch=4, Hc=Hc, D=D, dtype=dtype)
    b = st.add_sequence(total)
    bidx, pos = np.full(total, b), np.arange(total)
    k = randn(st.gen, (1, Hc, total, D), dtype)
    v = randn(st.gen, (1, Hc, total, D), dtype)
    q = randn(st.gen, (1, Hc * G, total, D), dtype)
    cache = st.cache
    dev = lambda a: torch.from_numpy(a)[None].to(DEV)
    if cut > 12:
        with pytest.raises(RuntimeError, match="still open"):
            cache.create_prefill_blockmask(dev(bidx[:cut]), dev(ids[:cut]), SOI, EOI, validate=True)
    cache.insert_kv(0, k[:, :, :cut].to(DEV), v[:, :, :cut].to(DEV), input_pos=dev(pos[:cut]), batch_idx=dev(bidx[:cut]))
    if 12 < cut <= 212:
        with pytest.raises(RuntimeError, match="open_spans"):
            cache.create_prefill_blockmask(dev(bidx[cut:]), dev(ids[cut:]), SOI, EOI, validate=True)
    mask = cache.create_prefill_blockmask(dev(bidx[cut:]), dev(ids[cut:]), SOI, EOI, open_spans=[b], validate=True)
    K, V = cache.insert_kv(0, k[:, :, cut:].to(DEV), v[:, :, cut:].to(DEV), input_pos=dev(pos[cut:]),
                           batch_idx=dev(bidx[cut:]))
    out, aux = A.compiled_flex_attn_prefill(q[:, :, cut:].to(DEV), K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
    eo, el = O.prefill_attention_packed(f64(q), f64(k), f64(v), bidx[None], ids[None], SOI, EOI)
    assert_close(out, aux.lse, eo[:, :, cut:], el[:, :, cut:], dtype)


def test_span_open_across_a_document_boundary_is_refused():
    ids = np.array([TXT] * 3 + [SOI] + [IMG] * 20 + [TXT] * 8 + [EOI] + [TXT] * 4)
    bidx = np.array([1] * 24 + [2] * 13)
    st = PagedState(22, n_pages=8, page_size=16, max_batch=4, Hc=1, D=64, dtype=torch.bfloat16)
    dev = lambda a: torch.from_numpy(a)[None].to(DEV)
    with pytest.raises(RuntimeError, match="still open"):
        st.cache.create_prefill_blockmask(dev(bidx), dev(ids), SOI, EOI, validate=True)
    # unchecked, the call returns as before (the mask of such a row is unspecified)
    st.cache.create_prefill_blockmask(dev(bidx), dev(ids), SOI, EOI, validate=False)
    # by default the report travels to the host behind the kernel and the next look at it raises
    st.cache.create_prefill_blockmask(dev(bidx), dev(ids), SOI, EOI)
    with pytest.raises(RuntimeError, match="previous create_prefill_blockmask.*still open"):
        st.cache.check_prefill_masks()
    st.cache.check_prefill_masks()  # looked at once
    st.cache.create_prefill_blockmask(dev(bidx), dev(ids), SOI, EOI)
    with pytest.raises(RuntimeError, match="still open"):
        st.cache.create_prefill_blockmask(dev(bidx[:20]), dev(ids[:20] * 0 + TXT), SOI, EOI)


def test_a_stray_end_of_image_token_is_masked_as_the_reference_masks_it_and_warns_late():
    """A sequence that sampled an end-of-image token of its own and is prefilled again after a preemption
    (paged_inference.py:1231-1237) carries an eoi with no span open.  The reference counts delimiters over the
    whole packed row (attention.py:75-96): nothing is inside a span while closed >= opened, so the stray token
    and the rows after it are causal -- and so is a LATER image span of the row, whose soi only brings the
    balance back to zero.  The kernel's limits are that mask; the default call does not wait and the report
    surfaces as a warning at the next look."""
    dtype, Hc, G, D, Pg = torch.bfloat16, 1, 2, 64, 16
    ids = np.array([TXT] * 5 + [EOI] + [TXT] * 6 + [SOI] + [IMG] * 10 + [EOI] + [TXT] * 7)
    L = len(ids)
    st = PagedState(23, n_pages=8, page_size=Pg, max_batch=3, Hc=Hc, D=D, dtype=dtype)
    b = st.add_sequence(L)
    bidx, pos = np.full(L, b), np.arange(L)
    dev = lambda a: torch.from_numpy(a)[None].to(DEV)
    with pytest.raises(RuntimeError, match="open_spans"):
        st.cache.create_prefill_blockmask(dev(bidx), dev(ids), SOI, EOI, validate=True)
    mask = st.cache.create_prefill_blockmask(dev(bidx), dev(ids), SOI, EOI)
    k, v, q = (randn(st.gen, (1, h, L, D), dtype) for h in (Hc, Hc, Hc * G))
    K, V = st.cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=dev(pos), batch_idx=dev(bidx))
    out, aux = A.compiled_flex_attn_prefill(q.to(DEV), K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
    # the reference's predicate on a dense grid (oracle: attention.py:75-96 OR document-causal)
    eo, el = O.prefill_attention_packed(f64(q), f64(k), f64(v), bidx[None], ids[None], SOI, EOI)
    assert_close(out, aux.lse, eo, el, dtype)
    assert (mask.row_hi.cpu().numpy() == np.arange(1, L + 1)).all()  # every row causal, the later span included
    with pytest.warns(RuntimeWarning, match="end-of-image"):
        st.cache.check_prefill_masks()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("G", [1, 2, 4, 8])
@pytest.mark.parametrize("P", [64, 16, 24], ids=["page-holds-tile", "small-page", "odd-page"])
def test_every_kernel_instance(dtype, D, G, P):
    """One small packed step per template instance (dtype, head_dim, query heads per cache head, and
    the three ways a key tile is staged: whole tiles from a page, row by row with a power-of-two page, row by
    row with any other page size): two sequences packed without padding, the second with an image span."""
    layout = layout_for([(1, 70, 0, 0), (2, 9, 60, 45)])
    ids, bidx, pos = repack(layout, 1)
    st = PagedState(40 + G, n_pages=24, page_size=P, max_batch=4, Hc=1, D=D, dtype=dtype)
    for slot in (1, 2):
        st.add_sequence(int((bidx == slot).sum()))
    q, k, v, out, lse = prefill_through_api(st, ids, bidx, pos, G, dtype, 1)
    eo, el = O.prefill_attention_packed(f64(q), f64(k), f64(v), bidx[None], ids[None], SOI, EOI)
    assert_close(out, lse, eo, el, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
@pytest.mark.parametrize("G,Hc", [(1, 16), (2, 8), (4, 4)])
@pytest.mark.parametrize("P", [128, 24], ids=["page-holds-tile", "odd-page"])
def test_head_dim_64_launch_of_a_workgroup_per_cu_and_more(dtype, G, Hc, P):
    """At head_dim 64 a launch that fills the GPU goes out as workgroups of four wavefronts (two to a CU):
    4096 rows x 16 query heads, 8 sequences packed without padding, image spans, prefixes already in pages.
    Sampled rows against the oracle; a padding stretch in the middle of the row."""
    gen = torch.Generator().manual_seed(64 + G)
    n_seq, chunk = 8, 500
    prefixes = [int(x) for x in torch.randint(0, 700, (n_seq,), generator=gen)]
    st = PagedState(64 + G, n_pages=sum(-(-(p + chunk) // P) for p in prefixes) + 8, page_size=P, max_batch=n_seq + 2,
                    Hc=Hc, D=64, dtype=dtype)
    st.cache.kv_cache.view(-1).normal_(generator=torch.Generator(device=DEV).manual_seed(1))
    bidx, lim = [], []
    for i, p in enumerate(prefixes):
        b = st.add_sequence(p + chunk)
        span = 200 if i % 2 else 0  # rows of the chunk's first `span` positions see the whole span
        bidx += [b] * chunk
        lim += [max(p + t + 1, p + span) for t in range(chunk)]
        if i == 3:
            bidx += [0] * 96
            lim += [0] * 96
    Lq = len(bidx)
    assert Lq == 4096
    q = randn(st.gen, (1, Hc * G, Lq, 64), dtype).to(DEV)
    pk, pv = st.pool_planes()
    bidx_t = torch.tensor(bidx, dtype=torch.int64, device=DEV)
    lim_t = torch.tensor(lim, dtype=torch.int32, device=DEV)
    out, lse = ops.paged_prefill(q, pk, pv, st.cache.page_table, bidx_t, lim_t, P)
    rows = np.arange(0, Lq, 29)
    eo, el = O.prefill_attention_paged(f64(q[:, :, rows]), f64(pk), f64(pv), st.mirror.page_table, np.array(bidx)[rows],
                                       None, np.array(lim)[rows], P)
    assert_close(out[:, :, rows], lse[:, :, rows], eo, el, dtype)
    pad = np.flatnonzero(np.array(bidx) == 0)
    assert not f64(out)[:, :, pad].any() and np.isneginf(f64(lse)[:, :, pad]).all()


# ---- bounded scores: the bf16 softmax without a running maximum -------------------------------------

def rms_normalised(gen, shape, dtype):
    """Rows of norm sqrt(D), as the model's weightless RMS norm leaves q and k (model.py:110-116), rounded to dtype."""
    x = torch.randn(shape, generator=gen, dtype=torch.float32)
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True))).to(dtype)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("G", [1, 2, 4, 8])
@pytest.mark.parametrize("P", [64, 16, 24], ids=["page-holds-tile", "small-page", "odd-page"])
def test_bounded_scores_every_kernel_instance(D, G, P):
    """The instances of the bf16 kernel that take the caller's score bound, one packed step each, through the
    drop-in callables: a cache that knows its q and k rows are normalised declares 1.1 * sqrt(D)."""
    dtype = torch.bfloat16
    layout = layout_for([(1, 70, 0, 0), (2, 9, 60, 45)])
    ids, bidx, pos = repack(layout, 1)
    st = PagedState(140 + G, n_pages=24, page_size=P, max_batch=4, Hc=1, D=D, dtype=dtype)
    for slot in (1, 2):
        st.add_sequence(int((bidx == slot).sum()))
    cache, L = st.cache, len(ids)
    cache.qk_normalised = True
    assert cache.score_bound(D, None) == pytest.approx(1.1 * D ** 0.5)
    dev = lambda a: torch.from_numpy(a)[None].to(DEV)
    mask = cache.create_prefill_blockmask(dev(bidx), dev(ids), SOI, EOI)
    k = rms_normalised(st.gen, (1, 1, L, D), dtype)
    v = randn(st.gen, (1, 1, L, D), dtype)
    q = rms_normalised(st.gen, (1, G, L, D), dtype)
    K, V = cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=dev(pos), batch_idx=dev(bidx))
    out, aux = A.compiled_flex_attn_prefill(q.to(DEV), K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
    eo, el = O.prefill_attention_packed(f64(q), f64(k), f64(v), bidx[None], ids[None], SOI, EOI)
    assert_close(out, aux.lse, eo, el, dtype, lse_atol=BOUNDED_LSE_ATOL)


@pytest.mark.parametrize("bound,peak", [(12.0, 11.0), (40.0, 38.0), (41.0, 38.0), (0.0, 38.0)])
def test_bounded_scores_over_a_wide_range(bound, peak):
    """Scores spread over +-peak (natural units): with the fixed reference point the probabilities span
    2^(+-peak * log2 e) and must survive in bf16 / fp32 without a running maximum; rows whose largest score is
    far below zero keep their precision.  A bound above the kernel's limit of 40, or none, takes the ordinary path."""
    dtype, D, P, L = torch.bfloat16, 128, 64, 300
    st = PagedState(150, n_pages=12, page_size=P, max_batch=3, Hc=1, D=D, dtype=dtype)
    b = st.add_sequence(L)
    gen = st.gen
    # keys along one direction with lengths that put scale * q.k anywhere in [-peak, peak]
    u = torch.randn(D, generator=gen)
    u /= u.norm()
    k = (u[None] * (torch.rand(L, 1, generator=gen) * 2 - 1) * 16 + 0.05 * torch.randn(L, D, generator=gen)).to(dtype)
    q = (u[None] * (torch.rand(L, 1, generator=gen) * 2 - 1) * (peak * D ** 0.5 / 16.2)
         + 0.05 * torch.randn(L, D, generator=gen)).to(dtype)
    assert (q.float() @ k.float().T).abs().max() / D ** 0.5 <= peak
    v = randn(gen, (L, D), dtype)
    bt, pt = torch.full((1, L), b, dtype=torch.int64), torch.arange(L)[None]
    st.cache.insert_kv(0, k.view(1, 1, L, D).to(DEV), v.view(1, 1, L, D).to(DEV), input_pos=pt.to(DEV), batch_idx=bt.to(DEV))
    lim = torch.arange(1, L + 1, dtype=torch.int32)
    pk, pv = st.pool_planes()
    q4 = q.view(1, 1, L, D)
    out, lse = ops.paged_prefill(q4.to(DEV), pk, pv, st.cache.page_table, bt.view(-1).to(DEV), lim.to(DEV), P,
                                 score_bound=bound)
    eo, el = O.prefill_attention_paged(f64(q4), f64(pk), f64(pv), st.mirror.page_table, bt.view(-1).numpy(), None,
                                       lim.numpy(), P)
    assert_close(out, lse, eo, el, dtype, lse_atol=BOUNDED_LSE_ATOL)


def test_bounded_scores_key_shares_and_f16():
    """A launch small enough to be cut along the keys (one 300-row chunk over a 3000-token prefix) with the bound
    declared: the shares' partial results all refer to the fixed point 0 and the merge pass combines them as
    before.  f16 ignores the bound."""
    D, P, prefix, chunk = 128, 128, 3000, 300
    for dtype in (torch.bfloat16, torch.float16):
        st = PagedState(151, n_pages=32, page_size=P, max_batch=3, Hc=2, D=D, dtype=dtype)
        b = st.add_sequence(prefix + chunk)
        L = prefix + chunk
        k = rms_normalised(st.gen, (1, 2, L, D), dtype)
        v = randn(st.gen, (1, 2, L, D), dtype)
        q = rms_normalised(st.gen, (1, 4, chunk, D), dtype)
        bt, pt = torch.full((1, L), b, dtype=torch.int64), torch.arange(L)[None]
        st.cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=pt.to(DEV), batch_idx=bt.to(DEV))
        lim = torch.arange(prefix + 1, L + 1, dtype=torch.int32)
        pk, pv = st.pool_planes()
        ws = st.cache.prefill_workspace(chunk, 4, D, 2, dtype)
        assert ws is not False
        rb = torch.full((chunk,), b, dtype=torch.int64)
        out, lse = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, rb.to(DEV), lim.to(DEV), P,
                                     workspace=ws, score_bound=1.1 * D ** 0.5)
        eo, el = O.prefill_attention_paged(f64(q), f64(pk), f64(pv), st.mirror.page_table, rb.numpy(), None, lim.numpy(), P)
        assert_close(out, lse, eo, el, dtype, lse_atol=BOUNDED_LSE_ATOL)


def test_cfg3_chunked_prefill_shape_with_the_score_bound():
    """BASELINE configs[2] at full size on the bounded path, the bound taken from the norms of the rows."""
    import bench

    case = bench.make_prefill_case("cfg3", device=DEV)
    case.append()
    assert case.score_bound > 0
    out, lse = case.attend()
    pk, pv = case.pool_k.float().cpu().numpy(), case.pool_v.float().cpu().numpy()
    bidx = case.batch_idx.cpu().numpy().reshape(-1)
    lim = case.row_limit.cpu().numpy()
    for s in (1, len(case.slots) - 2):
        rows = np.flatnonzero(bidx == case.slots[s])[3::11]
        eo, el = O.prefill_attention_paged(f64(case.q[:, :, rows]), pk, pv, case.page_table.cpu().numpy(),
                                           bidx[rows], None, lim[rows], case.page_size)
        assert_close(out[:, :, rows], lse[:, :, rows], eo, el, torch.bfloat16, lse_atol=BOUNDED_LSE_ATOL)


def test_the_measuring_kernel_runs_and_refuses_what_it_cannot_launch():
    """fp_probe_mfma_softmax is a measuring kernel (bench.py --overlap-probe), not an operator: every mode and
    wavefront count launches and fills its output, bad arguments come back as errors."""
    from falcon_perception_amd import _native as N

    lib = N.lib()
    out = torch.full((8 * 768,), float("nan"), dtype=torch.float32, device=DEV)
    stream = N.stream_ptr(out.device)
    for mode in (0, 1, 2):
        for waves in (1, 2, 3):
            out.fill_(float("nan"))
            N.check(lib.fp_probe_mfma_softmax(mode, waves, 8, 3, out.data_ptr(), out.numel(), stream), "probe")
            torch.cuda.synchronize()
            assert not torch.isnan(out[: 8 * 256 * waves]).any() or mode == 0  # mode 0 accumulates without bound
            assert torch.isnan(out[8 * 256 * waves:]).all()
    assert lib.fp_probe_mfma_softmax(2, 4, 8, 3, out.data_ptr(), out.numel(), stream) < 0
    assert lib.fp_probe_mfma_softmax(3, 1, 8, 3, out.data_ptr(), out.numel(), stream) < 0
    assert lib.fp_probe_mfma_softmax(2, 3, 9, 3, out.data_ptr(), out.numel(), stream) < 0  # out too small
