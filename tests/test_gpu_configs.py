"""GPU: the larger BASELINE.json configurations as parity cases.

cfg4  continuous-batching churn: mixed steps of 32 decode sequences and 4 prefill chunks of 1024
      tokens, 25 % of the live pages freed and reused between steps, page size 64, GQA 2.
cfg5  long-context decode on a pool sized to most of HBM (180 GB, shrunk to fit when the GPU
      has less free memory): batch 256, 32 q / 8 kv heads, contexts 4096 + U[256, 12288].
Full-size results are checked on sampled sequences / rows against the float64 oracle and through
properties that do not depend on size.
"""

import math

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from falcon_perception_amd.paged_attention import PagedKVCache
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, f64

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-2, 1e-2


def gathered_oracle_decode(q, pool_k, pool_v, page_table, slot, ctx, P):
    """Oracle for one sequence of a pool too large to copy to the host: gather the sequence on the
    GPU (bit-exact, tested separately), attend densely in float64 on the CPU."""
    dev = pool_k.device
    lens = torch.tensor([ctx], device=dev)
    slots = torch.tensor([slot], device=dev)
    K = ops.kv_gather(pool_k, page_table, slots, lens, P, ctx)[0]
    V = ops.kv_gather(pool_v, page_table, slots, lens, P, ctx)[0]
    return O.masked_attention_dense(f64(q), f64(K), f64(V), np.ones((1, ctx), dtype=bool))


def test_cfg4_continuous_batching_churn():
    gen = torch.Generator().manual_seed(4)
    dgen = torch.Generator(device=DEV).manual_seed(4)
    P, Hq, Hc, D, n_pages = 64, 16, 8, 128, 8192
    dtype = torch.bfloat16
    cache = PagedKVCache(n_pages, P, 64, Hc, D, 1, dtype, device=DEV)
    cache.free_pages = (torch.randperm(n_pages - 1, generator=gen) + 1).tolist()
    cache.kv_cache.view(-1).normal_(generator=dgen)  # stale bytes everywhere, as after long service
    pk, pv = cache.kv_cache[0, 0, 0], cache.kv_cache[0, 1, 0]
    rnd = lambda *shape: torch.randn(shape, generator=dgen, device=DEV, dtype=torch.float32).to(dtype)

    def admit(length):
        b = cache.allocate()
        cache.reserve(b, torch.tensor([b], device=DEV), length)
        return b

    def fill(slot, start, n):
        """Append n random rows at positions start.. of a sequence (packed prefill append)."""
        k, v = rnd(1, Hc, n, D), rnd(1, Hc, n, D)
        bidx = torch.full((1, n), slot, dtype=torch.int64, device=DEV)
        pos = torch.arange(start, start + n, dtype=torch.int64, device=DEV)[None]
        cache.insert_kv(0, k, v, input_pos=pos, batch_idx=bidx)

    ctx = {}
    for L in torch.randint(512, 8193, (32,), generator=gen).tolist():
        if not cache.can_reserve(L + 8):
            break
        s = admit(L + 8)
        fill(s, 0, L)
        ctx[s] = L
    assert len(ctx) >= 24

    for step in range(3):
        # --- 4 prefill chunks of 1024 tokens: 2 fresh sequences whose first 512 tokens are an image
        #     span, 2 sequences continuing after a 2048-token prefix already in pages
        chunks = []
        for kind in ("fresh", "fresh", "cont", "cont"):
            if kind == "fresh":
                s = admit(1024)
                lim = [max(t + 1, 512) for t in range(1024)]
                start = 0
            else:
                s = admit(2048 + 1024)
                fill(s, 0, 2048)
                lim = [2048 + t + 1 for t in range(1024)]
                start = 2048
            chunks.append((s, start, lim))
        bidx = torch.cat([torch.full((1024,), s, dtype=torch.int64) for s, _, _ in chunks])[None].to(DEV)
        pos = torch.cat([torch.arange(st, st + 1024, dtype=torch.int64) for _, st, _ in chunks])[None].to(DEV)
        lim = torch.tensor([x for _, _, l in chunks for x in l], dtype=torch.int32, device=DEV)
        k, v, q = rnd(1, Hc, 4096, D), rnd(1, Hc, 4096, D), rnd(1, Hq, 4096, D)
        cache.insert_kv(0, k, v, input_pos=pos, batch_idx=bidx)
        out, lse = ops.paged_prefill(q, pk, pv, cache.page_table, bidx, lim, P)
        rows = np.arange(0, 4096, 61)  # sampled rows of every chunk
        pt = cache.page_table.cpu().numpy()
        eo, el = O.prefill_attention_paged(f64(q[:, :, rows]), pk.float().cpu().numpy(), pv.float().cpu().numpy(), pt,
                                           bidx.cpu().numpy().reshape(-1)[rows], None, lim.cpu().numpy()[rows], P)
        np.testing.assert_allclose(f64(out[:, :, rows]), eo, atol=ATOL, rtol=RTOL)
        np.testing.assert_allclose(f64(lse[:, :, rows]), el, atol=2e-3, rtol=RTOL)

        # --- decode step over every running sequence: fused append + attention
        slots = sorted(ctx)
        B = len(slots)
        bt = torch.tensor(slots, dtype=torch.int64, device=DEV)
        pt_ = torch.tensor([ctx[s] for s in slots], dtype=torch.int32, device=DEV)
        k1, v1, q1 = rnd(B, Hc, 1, D), rnd(B, Hc, 1, D), rnd(B, Hq, 1, D)
        o1, l1 = ops.paged_decode(q1, pk, pv, cache.page_table, bt, pt_, P, 8192 + 64, k_new=k1, v_new=v1)
        for i in range(0, B, 5):
            s = slots[i]
            eo, el = gathered_oracle_decode(q1[i], pk, pv, cache.page_table, s, ctx[s] + 1, P)
            np.testing.assert_allclose(f64(o1[i]), eo, atol=ATOL, rtol=RTOL)
            np.testing.assert_allclose(f64(l1[i]), el, atol=2e-3, rtol=RTOL)
            # the appended row is in its slot, bit for bit
            page = cache.page_table_cpu[s][ctx[s] // P]
            assert torch.equal(pk[:, page * P + ctx[s] % P].view(torch.int16), k1[i, :, 0].view(torch.int16))
        for s in slots:
            ctx[s] += 1

        # --- churn: the chunk sequences leave, a quarter of the decode sequences are replaced
        for s, _, _ in chunks:
            cache.erase(s)
        leaving = [slots[i] for i in torch.randperm(B, generator=gen)[: B // 4].tolist()]
        for s in leaving:
            cache.erase(s)
            del ctx[s]
        for L in torch.randint(512, 8193, (len(leaving),), generator=gen).tolist():
            if cache.can_reserve(L + 8):
                s = admit(L + 8)
                fill(s, 0, L)
                ctx[s] = L
        live = [p for s in ctx for p in cache.page_table_cpu[s]]
        assert len(live) == len(set(live)) and 0 not in live
        assert len(live) + cache.num_free_pages == n_pages - 1


@pytest.mark.parametrize("name", ["cfg2", "cfg2d64", "cfg2f32", "cfg2x", "cfg2xs", "cfg4d"])
def test_decode_workloads_of_the_bench_at_full_size(name):
    """The decode workloads bench.py reports (BASELINE configs[1] and its variants: head_dim 64, fp32, the
    engine's 16-head cache read plainly and with V once per group; the decode part of configs[3]), fused
    append included: sampled sequences against the float64 oracle, and the step with the step's plan against
    the step without, bit for bit, pool included."""
    import bench

    case = bench.make_decode_case(name, device=DEV)
    c = case.cfg
    if c.get("kv_rep", 1) > 1:  # the V copies of a group are identical in the engine's cache
        rep, pv = c["kv_rep"], case.pool_v
        pv.copy_(pv.view(-1, rep, *pv.shape[1:])[:, :1].expand(-1, rep, *pv.shape[1:]).reshape(pv.shape).clone())
        case.v_new.copy_(case.v_new.view(c["B"], -1, rep, 1, c["D"])[:, :, :1].expand(-1, -1, rep, -1, -1)
                         .reshape(case.v_new.shape).clone())
    before = case.cache.kv_cache.clone()
    assert case.planned
    rec = case.plan.view(torch.int32).view(-1, 128 + 1024)[0].cpu()
    assert rec[0] >= 1 and rec[1] == c["B"]  # the launch is cut evenly and chunk 0 has its record
    out, lse = (t.clone() for t in case.run_fused())
    after = case.cache.kv_cache.clone()
    case.cache.kv_cache.copy_(before)
    case.planned = False
    out0, lse0 = case.run_fused()
    assert torch.equal(out, out0) and torch.equal(lse, lse0)
    assert torch.equal(case.cache.kv_cache, after)
    atol, rtol = (2e-5, 2e-5) if case.q.dtype == torch.float32 else (ATOL, RTOL)
    order = np.argsort(case.lens)
    for i in [order[0], order[-1], order[len(order) // 2], 0, c["B"] - 1]:
        slot = int(case.batch_idx[i])
        eo, el = gathered_oracle_decode(case.q[i], case.pool_k, case.pool_v, case.page_table, slot, case.lens[i] + 1,
                                        case.page_size)
        np.testing.assert_allclose(f64(out[i]), eo, atol=atol, rtol=rtol)
        np.testing.assert_allclose(f64(lse[i]), el, atol=max(atol * 0.1, 1e-5), rtol=rtol)
        # the appended row is in its slot, bit for bit
        L = case.lens[i]
        page = int(case.page_table[slot, L // case.page_size])
        at = page * case.page_size + L % case.page_size
        view = torch.int32 if case.q.dtype == torch.float32 else torch.int16
        assert torch.equal(case.pool_k[:, at].view(view), case.k_new[i, :, 0].view(view))
        assert torch.equal(case.pool_v[:, at].view(view), case.v_new[i, :, 0].view(view))


@pytest.mark.bigmem
def test_cfg5_long_context_decode_on_a_pool_sized_to_hbm():
    import bench

    free, total = torch.cuda.mem_get_info()
    budget = min(180.0, (free - 24e9) / 1e9)
    # a box that cannot hold a 30 GB pool is not an MI355X to itself: fail, a skip would pass silently
    assert budget >= 30, f"only {free / 1e9:.0f} GB of HBM free: cfg5 needs a pool of at least 30 GB"
    case = bench.make_decode_case("cfg5", device=DEV, hbm_budget_gb=budget)
    c = case.cfg
    assert case.pool_k.numel() * 2 > 2**32  # byte offsets inside one plane need 64 bits
    out, lse = (t.clone() for t in case.run_fused())  # reads the step's plan
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    case.planned = False
    out0, lse0 = case.run_fused()  # the new rows are in the pool already: the same rows are stored again
    assert torch.equal(out, out0) and torch.equal(lse, lse0)
    # sampled sequences against the oracle: shortest, longest, and a few in between
    order = np.argsort(case.lens)
    for i in [order[0], order[-1], order[len(order) // 2], 0, c["B"] - 1]:
        slot = int(case.batch_idx[i])
        eo, el = gathered_oracle_decode(case.q[i], case.pool_k, case.pool_v, case.page_table, slot, case.lens[i] + 1,
                                        case.page_size)
        np.testing.assert_allclose(f64(out[i]), eo, atol=ATOL, rtol=RTOL)
        np.testing.assert_allclose(f64(lse[i]), el, atol=2e-3, rtol=RTOL)
    # split-count invariance on the whole batch
    o2, l2 = ops.paged_decode(case.q, case.pool_k, case.pool_v, case.page_table, case.batch_idx, case.input_pos,
                              case.page_size, case.max_context, split_tokens=512)
    np.testing.assert_allclose(l2.cpu().numpy(), lse.cpu().numpy(), atol=1e-4, rtol=1e-5)
    np.testing.assert_allclose(f64(o2), f64(out), atol=8e-3, rtol=8e-3)


@pytest.mark.parametrize("name", ["cfg3w", "cfg3wx", "cfg3wd64"])
@pytest.mark.parametrize("bounded", [False, True], ids=["running-maximum", "score-bound"])
def test_whole_sequence_prefill_at_full_size(name, bounded):
    """The prefill step the reference's engine runs (whole sequences packed, each padded to 128,
    paged_inference.py:637-672) at the size the bench times: 8 sequences of an image span of U[256, 4096] tokens
    plus 512 text tokens, 23040 packed rows, 16 query heads; on 8 cached heads, on the engine's 16, at head_dim 64.
    Everything goes through the drop-in: the mask from the token ids (`create_prefill_blockmask` -> row-limit
    kernel -> `row_limit`), `insert_kv`, `compiled_flex_attn_prefill`.  Checked: the limits against the oracle's
    (and against the ones the bench writes by hand), the pool against the rows, and sampled rows of three
    sequences -- inside the span (first, middle, last), the end-of-image row, the first and the last text row --
    against the float64 oracle."""
    import bench
    from torch.nn.attention.flex_attention import AuxRequest

    from falcon_perception_amd import attention as A
    from tests.test_gpu_prefill import BOUNDED_LSE_ATOL

    case = bench.make_prefill_case(name, device=DEV)
    cache = case.cache
    bidx = case.batch_idx.cpu().numpy().reshape(-1)
    ids = case.input_ids.cpu().numpy().reshape(-1)
    pos = case.input_pos.cpu().numpy().reshape(-1)
    L = len(ids)
    assert L == 23040 and case.q.shape[2] == L

    mask = cache.create_prefill_blockmask(case.batch_idx, case.input_ids, bench.SOI_ID, bench.EOI_ID)
    hi, status = O.chunk_row_limits(bidx, ids, bench.SOI_ID, bench.EOI_ID)
    assert status == 0
    assert np.array_equal(mask.row_hi.cpu().numpy(), hi)
    limits = (pos + hi - np.arange(L)).astype(np.int32)  # logical: position + reach beyond the row
    assert np.array_equal(mask.row_limit(case.input_pos, 0).cpu().numpy(), limits)
    real = bidx != 0
    assert np.array_equal(case.row_limit.cpu().numpy()[real], limits[real])

    if bounded:
        cache.score_bound = lambda head_dim, scale: case.score_bound  # a bound that holds for these N(0, 1) rows
    K, V = cache.insert_kv(0, case.k_new, case.v_new, input_pos=case.input_pos, batch_idx=case.batch_idx)
    out, aux = A.compiled_flex_attn_prefill(case.q, K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
    cache.check_prefill_masks()

    pk, pv = case.pool_k.float().cpu().numpy(), case.pool_v.float().cpu().numpy()
    pt = case.page_table.cpu().numpy()
    rows = []
    for s in (0, 3, len(case.slots) - 1):
        r = np.flatnonzero(bidx == case.slots[s])
        p = case.prefixes[s]
        rows += [r[0], r[p // 2], r[p - 1], r[p], r[p + 1], r[-1]]
        # the rows just appended are the keys the attention read
        slots_of = pt[case.slots[s], pos[r] // case.page_size] * case.page_size + pos[r] % case.page_size
        assert np.array_equal(pk[:, slots_of], case.k_new[0][:, r].float().cpu().numpy())
    rows = np.array(sorted(rows))
    eo, el = O.prefill_attention_paged(f64(case.q[:, :, rows]), pk, pv, pt, bidx[rows], None, limits[rows], case.page_size)
    go, gl = f64(out[:, :, rows]), f64(aux.lse[:, :, rows])
    np.testing.assert_allclose(go, eo, atol=ATOL, rtol=RTOL)
    np.testing.assert_allclose(gl, el, atol=BOUNDED_LSE_ATOL if bounded else 2e-3, rtol=RTOL)
    pad = np.flatnonzero(~real)
    assert not f64(out[:, :, pad]).any() and np.isneginf(f64(aux.lse[:, :, pad])).all()
