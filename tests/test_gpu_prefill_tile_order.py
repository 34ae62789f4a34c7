"""GPU: the order of a prefill launch's workgroups (fp_paged_prefill_tile_order).

The order only decides which query tile a workgroup row works on: the ranking itself is checked against numpy,
and every launch that takes an order must return the bits of the same launch without one.
"""

import numpy as np
import pytest
import torch
from torch.nn.attention.flex_attention import AuxRequest

from falcon_perception_amd import attention as A
from falcon_perception_amd import ops
from tests.gpu_cases import DEV, PagedState, randn
from tests.test_gpu_prefill import EOI, SOI, layout_for, repack

pytestmark = pytest.mark.gpu


def packed_chunks(seed, n_seq, chunk, max_prefix, P, Hc, D, dtype, pad_after=()):
    """n_seq chunks of `chunk` rows over paged prefixes of random length; every other chunk starts with a
    bidirectional stretch; padding rows after the sequences named in `pad_after`."""
    gen = torch.Generator().manual_seed(seed)
    prefixes = [int(x) for x in torch.randint(0, max_prefix + 1, (n_seq,), generator=gen)]
    st = PagedState(seed, n_pages=sum(-(-(p + chunk) // P) for p in prefixes) + 8, page_size=P, max_batch=n_seq + 2, Hc=Hc,
                    D=D, dtype=dtype)
    st.cache.kv_cache.view(-1).normal_(generator=torch.Generator(device=DEV).manual_seed(seed))
    bidx, lim = [], []
    for i, p in enumerate(prefixes):
        b = st.add_sequence(p + chunk)
        span = chunk // 3 if i % 2 else 0
        bidx += [b] * chunk
        lim += [max(p + t + 1, p + span) for t in range(chunk)]
        if i in pad_after:
            bidx += [0] * 96
            lim += [0] * 96
    return st, torch.tensor(bidx, dtype=torch.int64, device=DEV), torch.tensor(lim, dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("tile_rows", [32, 64, 128, 256])
@pytest.mark.parametrize("Lq", [1, 777, 4096, 23040])
def test_the_order_is_the_tiles_by_decreasing_key_range(tile_rows, Lq):
    """order[i] = the tile of rank i: a permutation of the tiles, key tiles (64 keys) non-increasing along it, the
    later tile first among equals; a tile's key range is the largest limit of its rows, padding rows not counted."""
    rng = np.random.default_rng(Lq + tile_rows)
    lim = rng.integers(0, 5000, Lq).astype(np.int32)
    bidx = rng.integers(0, 4, Lq).astype(np.int64)  # a quarter of the rows are padding (sequence 0)
    lim[rng.integers(0, Lq, max(Lq // 50, 1))] = 0
    order, rows = ops.prefill_tile_order(torch.from_numpy(bidx).to(DEV), torch.from_numpy(lim).to(DEV), tile_rows)
    assert rows == tile_rows
    n_tiles = -(-Lq // tile_rows)
    got = order.cpu().numpy()
    assert sorted(got.tolist()) == list(range(n_tiles))
    seen = np.where(bidx != 0, lim, 0)
    seen = np.concatenate([seen, np.zeros(n_tiles * tile_rows - Lq, dtype=seen.dtype)]).reshape(n_tiles, tile_rows)
    kt = (seen.max(axis=1) + 63) // 64
    want = sorted(range(n_tiles), key=lambda t: (-kt[t], -t))
    assert got.tolist() == want


def test_tile_order_arguments_are_checked():
    b = torch.ones(100, dtype=torch.int64, device=DEV)
    lim = torch.ones(100, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="tile_rows"):
        ops.prefill_tile_order(b, lim, 48)
    with pytest.raises(RuntimeError, match="int64"):
        ops.prefill_tile_order(b.int(), lim, 64)
    big = torch.ones(4097 * 32, dtype=torch.int64, device=DEV)
    with pytest.raises(RuntimeError, match="query tiles"):
        ops.prefill_tile_order(big, big.int(), 32)
    assert ops.prefill_tile_rows(4096, 16, 8, 128, torch.bfloat16) == 128
    assert ops.prefill_tile_rows(4096, 16, 8, 64, torch.bfloat16) == 64   # four-wavefront workgroups
    assert ops.prefill_tile_rows(4096, 16, 2, 64, torch.bfloat16) == 32   # eight query heads per cache head: eight wavefronts
    assert ops.prefill_tile_rows(4096, 16, 16, 128, torch.float16) == 256
    assert ops.prefill_tile_rows(4096, 16, 8, 128, torch.float32) == 0    # the fp32 kernel takes no order


@pytest.mark.parametrize("dtype,D,G,Hc,P", [
    (torch.bfloat16, 64, 2, 8, 128), (torch.bfloat16, 64, 1, 8, 24), (torch.float16, 64, 4, 4, 64),
    (torch.bfloat16, 64, 8, 2, 64), (torch.bfloat16, 128, 2, 8, 128), (torch.float16, 128, 1, 4, 16)], ids=str)
@pytest.mark.parametrize("bounded", [False, True], ids=["running-maximum", "score-bound"])
def test_a_launch_with_an_order_returns_the_bits_of_the_launch_without(dtype, D, G, Hc, P, bounded):
    """Six chunks of 500 rows over prefixes of up to 1500 tokens, padding rows in the middle: four- and
    eight-wavefront workgroups, both softmax paths.  An order made for another tile size is not used (same bits
    again); an order full of values that are no tiles does not make the launch read outside its rows."""
    st, bidx, lim = packed_chunks(7 + G, 6, 500, 1500, P, Hc, D, dtype, pad_after=(2,))
    Lq = bidx.numel()
    q = randn(st.gen, (1, Hc * G, Lq, D), dtype).to(DEV)
    pk, pv = st.pool_planes()
    bound = 0.0
    if bounded:
        bound = float(q.float().norm(dim=-1).max()) * float(pk.float().norm(dim=-1).max()) / D ** 0.5
    kw = dict(workspace=False, score_bound=bound)
    ref = ops.paged_prefill(q, pk, pv, st.cache.page_table, bidx, lim, P, **kw)
    rows = ops.prefill_tile_rows(Lq, Hc * G, Hc, D, dtype)
    order = ops.prefill_tile_order(bidx, lim, rows)
    got = ops.paged_prefill(q, pk, pv, st.cache.page_table, bidx, lim, P, tile_order=order, **kw)
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    other = 32 if rows != 32 else 64
    foreign = ops.prefill_tile_order(bidx, lim, other)
    got = ops.paged_prefill(q, pk, pv, st.cache.page_table, bidx, lim, P, tile_order=foreign, **kw)
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    junk = (torch.full_like(order[0], -7), rows)
    junk[0][::2] = 1 << 20
    ops.paged_prefill(q, pk, pv, st.cache.page_table, bidx, lim, P, tile_order=junk, **kw)
    torch.cuda.synchronize()


def test_the_order_with_the_launch_cut_along_the_keys():
    """One sequence's chunk (few workgroups): with a workspace the launch is cut along the keys and keeps the
    eight-wavefront tile size also at head_dim 64; the order made for that size is taken, same bits."""
    dtype, D, G, Hc, P = torch.bfloat16, 64, 2, 8, 128
    st, bidx, lim = packed_chunks(31, 1, 512, 3000, P, Hc, D, dtype)
    Lq = bidx.numel()
    q = randn(st.gen, (1, Hc * G, Lq, D), dtype).to(DEV)
    pk, pv = st.pool_planes()
    need = ops.prefill_workspace_bytes(Lq, Hc * G, Hc, D, dtype)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    rows = ops.prefill_tile_rows(Lq, Hc * G, Hc, D, dtype, need)
    assert rows == 128 and ops.prefill_tile_rows(Lq, Hc * G, Hc, D, dtype, 0) == 64
    ref = ops.paged_prefill(q, pk, pv, st.cache.page_table, bidx, lim, P, workspace=ws)
    got = ops.paged_prefill(q, pk, pv, st.cache.page_table, bidx, lim, P, workspace=ws,
                            tile_order=ops.prefill_tile_order(bidx, lim, rows))
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])


@pytest.mark.parametrize("D,calls_per_step", [(64, 1), (128, 0)])
def test_the_drop_in_ranks_the_tiles_once_per_step_at_head_dim_64(monkeypatch, D, calls_per_step):
    """compiled_flex_attn_prefill: the first layer of a step has the order written, the layers after it reuse it;
    a new step (new positions) ranks again; at head_dim 128 no order is made.  Results equal the library call
    without an order."""
    dtype, Hc, G, P, layers = torch.bfloat16, 4, 2, 64, 3
    layout = layout_for([(1, 5, 150, 40), (2, 0, 60, 200), (3, 131, 0, 0)])
    ids, bidx, pos = repack(layout, 128)
    st = PagedState(77, n_pages=32, page_size=P, max_batch=6, Hc=Hc, D=D, dtype=dtype, n_layers=layers)
    for slot in (1, 2, 3):
        st.add_sequence(int((bidx == slot).sum()))
    cache = st.cache
    t_ids, t_b = torch.from_numpy(ids)[None].to(DEV), torch.from_numpy(bidx)[None].to(DEV)
    made = []
    real = ops.prefill_tile_order
    monkeypatch.setattr(ops, "prefill_tile_order", lambda *a, **k: (made.append(1), real(*a, **k))[1])
    for step_no in range(2):
        t_p = torch.from_numpy(pos)[None].to(DEV).clone()
        mask = cache.create_prefill_blockmask(t_b, t_ids, SOI, EOI)
        made.clear()
        for layer in range(layers):
            L = len(ids)
            k, v = randn(st.gen, (1, Hc, L, D), dtype).to(DEV), randn(st.gen, (1, Hc, L, D), dtype).to(DEV)
            q = randn(st.gen, (1, Hc * G, L, D), dtype).to(DEV)
            K, V = cache.insert_kv(layer, k, v, input_pos=t_p, batch_idx=t_b)
            out, aux = A.compiled_flex_attn_prefill(q, K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
            pk, pv = cache.kv_cache[layer, 0, 0], cache.kv_cache[layer, 1, 0]
            eo, el = ops.paged_prefill(q, pk, pv, cache.page_table, t_b.reshape(-1), mask._row_limit, P,
                                       workspace=cache.prefill_workspace(L, Hc * G, D, Hc, dtype))
            assert torch.equal(out, eo) and torch.equal(aux.lse, el)
        assert len(made) == calls_per_step
