"""GPU parity: the decode step plan (fp_paged_decode_plan).

A plan holds, per chunk of the even cut, the pieces and page ids every layer of a decode step would otherwise
work out again from the positions, the slots and the page table.  It changes when a workgroup learns its
work, never the work: every launch that uses a plan must return the bits of the same launch without one
(which the other decode tests hold against the float64 oracle; the first test here does so as well).
"""

import numpy as np
import pytest
import torch
from torch.nn.attention.flex_attention import AuxRequest, BlockMask

from falcon_perception_amd import attention as A
from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, f64, randn

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: (2e-2, 1e-2), torch.float16: (2e-3, 2e-3), torch.float32: (2e-5, 2e-5)}
REC, PAGES = 128, 1024  # ints of a chunk's record and of its page list


def new_plan(fill=0):
    return torch.full((ops.decode_plan_bytes(),), fill, dtype=torch.uint8, device=DEV)


def records(plan):
    return plan.view(torch.int32).view(-1, REC + PAGES).cpu().numpy()


def decode(st, q, pos, **kw):
    pk, pv = st.pool_planes()
    bidx = kw.pop("bidx", None)
    if bidx is None:
        bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    return ops.paged_decode(q, pk, pv, st.cache.page_table, bidx, pos, st.P, **kw)


def flat_state(seed, B, Hc, D, P, ctx, dtype, rep=1, lens=None):
    """B sequences on Hc * rep cached heads, contexts below ctx, some empty, one full; V copies of a group
    identical where rep > 1."""
    gen = torch.Generator().manual_seed(seed)
    if lens is None:
        lens = torch.randint(0, ctx - 1, (B,), generator=gen).tolist()
        lens[0], lens[1], lens[2] = ctx - 1, 0, 64
    st = PagedState(seed, n_pages=sum(-(-(L + 1) // P) for L in lens) + 8, page_size=P, max_batch=B + 2, Hc=Hc * rep,
                    D=D, dtype=dtype)
    for L in lens:
        st.add_sequence(L + 1)
    st.lens = lens
    st.prefill_random()
    if rep > 1:
        _, pv = st.pool_planes()
        pv.copy_(pv.view(Hc, rep, *pv.shape[1:])[:, :1].expand(Hc, rep, *pv.shape[1:]).reshape(pv.shape).clone())
    return st


@pytest.mark.parametrize("dtype,D,P,G,rep", [
    (torch.bfloat16, 128, 64, 2, 1), (torch.bfloat16, 64, 24, 4, 1), (torch.float32, 64, 16, 1, 1),
    (torch.float16, 128, 48, 8, 1), (torch.bfloat16, 128, 64, 2, 2), (torch.bfloat16, 64, 16, 4, 4)], ids=str)
def test_a_planned_step_returns_the_bits_of_the_unplanned_one(dtype, D, P, G, rep):
    """4 cache heads x 96 sequences x 8 splits, more workgroups than the GPU holds at once, so the launch is
    cut evenly and reads the plan.  Fused append, aligned and odd pages, a cache expanded to one head per query
    head; the pool after the step, out and lse against the same step without a plan, and against the oracle."""
    B, Hc, split, ctx = 96, 4, 64, 512
    st = flat_state(80 + G, B, Hc, D, P, ctx, dtype, rep)
    q = randn(st.gen, (B, Hc * G, 1, D), dtype).to(DEV)
    k_new = randn(st.gen, (B, Hc * rep, 1, D), dtype).to(DEV)
    v_new = randn(st.gen, (B, Hc, 1, D), dtype).repeat_interleave(rep, dim=1).to(DEV)
    pos = torch.tensor(st.lens, dtype=torch.int32, device=DEV)
    kw = dict(max_context=ctx, split_tokens=split, kv_rep=rep)
    before = st.cache.kv_cache.clone()
    out0, lse0 = decode(st, q, pos, k_new=k_new, v_new=v_new, **kw)
    pool0 = st.cache.kv_cache.clone()
    st.cache.kv_cache.copy_(before)
    plan = new_plan()
    decode(st, q, pos, phase="plan", plan=plan, **kw)
    rec = records(plan)
    n_chunks = 2 * torch.cuda.get_device_properties(0).multi_processor_count // Hc
    assert (rec[:n_chunks, 1] == B).all() and (rec[:n_chunks, 2] == n_chunks).all() and (rec[:n_chunks, 3] == ctx).all()
    assert (rec[:n_chunks, 0] >= 0).all() and rec[:n_chunks, 0].sum() >= B - 2  # every sequence with a key has a piece
    out1, lse1 = decode(st, q, pos, k_new=k_new, v_new=v_new, plan=plan, **kw)
    assert torch.equal(out1, out0) and torch.equal(lse1, lse0)
    assert torch.equal(st.cache.kv_cache, pool0)
    # the passes called separately, without the append (the rows are in the pool now)
    ws = torch.empty(ops.decode_workspace_bytes(B, Hc * G, D, ctx, split), dtype=torch.uint8, device=DEV)
    ref = decode(st, q, pos, workspace=ws, **kw)
    ws.fill_(0xA5)
    decode(st, q, pos, workspace=ws, phase="partial", plan=plan, **kw)
    got = decode(st, q, pos, workspace=ws, phase="merge", plan=plan, **kw)
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    pk, pv = st.pool_planes()
    eo, el = O.decode_attention(f64(q), f64(pk), f64(pv), st.mirror.page_table, st.slots, np.array(st.lens), P)
    atol, rtol = TOL[dtype]
    np.testing.assert_allclose(f64(out1), eo, atol=atol, rtol=rtol)
    np.testing.assert_allclose(f64(lse1), el, atol=max(atol * 0.1, 1e-5), rtol=rtol)


@pytest.mark.parametrize("pos_dtype", [torch.int32, torch.int64], ids=str)
def test_masked_sequences_and_foreign_slots_under_a_plan(pos_dtype):
    """Sequences the launch must skip - position -1 (a padded row), a slot outside the page table, a position at
    or beyond max_context - have no piece in the plan either: out 0 / lse -inf for the first two, the context
    clamped for the third, nothing appended for any of them; bit for bit what the launch without a plan does.
    Positions as int32 and as int64 (what the engine passes)."""
    dtype, B, Hc, G, D, P, split, ctx = torch.bfloat16, 80, 8, 2, 128, 32, 64, 384
    st = flat_state(99, B, Hc, D, P, ctx - 2, dtype)
    q = randn(st.gen, (B, Hc * G, 1, D), dtype).to(DEV)
    k_new = randn(st.gen, (B, Hc, 1, D), dtype).to(DEV)
    v_new = randn(st.gen, (B, Hc, 1, D), dtype).to(DEV)
    pos = torch.tensor(st.lens, dtype=pos_dtype, device=DEV)
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    pos[5] = -1
    bidx[9] = B + 40      # beyond max_batch
    bidx[11] = -3
    pos[13] = ctx + 7     # beyond what the launch was sized for
    kw = dict(max_context=ctx, split_tokens=split, bidx=bidx)
    before = st.cache.kv_cache.clone()
    ref = decode(st, q, pos, k_new=k_new, v_new=v_new, **kw)
    pool_ref = st.cache.kv_cache.clone()
    st.cache.kv_cache.copy_(before)
    plan = new_plan()
    decode(st, q, pos, phase="plan", plan=plan, **kw)
    got = decode(st, q, pos, k_new=k_new, v_new=v_new, plan=plan, **kw)
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    assert torch.equal(st.cache.kv_cache, pool_ref)
    for i in (5, 9, 11):
        assert not got[0][i].any() and torch.isneginf(got[1][i]).all()
    assert torch.isfinite(got[1][13]).all()
    changed = (pool_ref != before).flatten(0, -3).any(-1)  # per pool slot, any layer / plane / head
    assert int(changed.sum()) == (B - 4) * 2 * Hc  # one K and one V row per head of every sequence that appended


def test_a_plan_of_another_launch_and_a_buffer_never_planned_are_ignored():
    """A workgroup uses a record only if it carries the launch's batch, chunk count and max_context; anything
    else (a plan made for one sequence more, for another max_context, a buffer of zeros or of 0xA5) leaves the
    launch working its cut out itself."""
    dtype, B, Hc, G, D, P, split, ctx = torch.bfloat16, 80, 8, 2, 128, 32, 64, 384
    st = flat_state(91, B, Hc, D, P, ctx, dtype)
    q = randn(st.gen, (B, Hc * G, 1, D), dtype).to(DEV)
    pos = torch.tensor(st.lens, dtype=torch.int32, device=DEV)
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    kw = dict(max_context=ctx, split_tokens=split)
    ref = decode(st, q[:-1], pos[:-1], bidx=bidx[:-1], **kw)
    plan = new_plan()
    decode(st, q, pos, phase="plan", plan=plan, **kw)  # for B sequences
    assert records(plan)[0, 1] == B
    for stale in (plan, new_plan(0), new_plan(0xA5)):
        got = decode(st, q[:-1], pos[:-1], bidx=bidx[:-1], plan=stale, **kw)
        assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    wide = dict(max_context=ctx + 64, split_tokens=split)
    ref_w = decode(st, q, pos, **wide)
    got_w = decode(st, q, pos, plan=plan, **wide)
    assert torch.equal(got_w[0], ref_w[0]) and torch.equal(got_w[1], ref_w[1])


def test_a_plan_made_from_other_positions_fails_loudly():
    """The contract is that positions and slots do not change between the plan and its launches.  If they did
    (same batch, same shapes, so the workgroups accept the records), the merge pass finds the hash of the
    step's positions and slots different from the plan's and stores NaN in every row of out and lse."""
    dtype, B, Hc, G, D, P, split, ctx = torch.bfloat16, 80, 8, 2, 128, 32, 64, 384
    st = flat_state(98, B, Hc, D, P, ctx - 2, dtype)
    q = randn(st.gen, (B, Hc * G, 1, D), dtype).to(DEV)
    pos = torch.tensor(st.lens, dtype=torch.int32, device=DEV)
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    kw = dict(max_context=ctx, split_tokens=split)
    plan = new_plan()
    decode(st, q, pos, phase="plan", plan=plan, **kw)
    # one sequence a token further than planned
    moved = pos.clone()
    moved[7] += 1
    out, lse = decode(st, q, moved, plan=plan, **kw)
    assert torch.isnan(out.float()).all() and torch.isnan(lse).all()
    # two sequences in each other's slots (the sums of the positions and of the slots are what they were)
    swapped = bidx.clone()
    swapped[3], swapped[4] = bidx[4], bidx[3]
    out, lse = decode(st, q, pos, bidx=swapped, plan=plan, **kw)
    assert torch.isnan(out.float()).all() and torch.isnan(lse).all()
    # the passes called separately report it as well
    ws = torch.empty(ops.decode_workspace_bytes(B, Hc * G, D, ctx, split), dtype=torch.uint8, device=DEV)
    decode(st, q, moved, workspace=ws, phase="partial", plan=plan, **kw)
    out, lse = decode(st, q, moved, workspace=ws, phase="merge", plan=plan, **kw)
    assert torch.isnan(out.float()).all() and torch.isnan(lse).all()
    # planned anew for what the step holds, the launch is a result again
    decode(st, q, moved, phase="plan", plan=plan, **kw)
    out, lse = decode(st, q, moved, plan=plan, **kw)
    ref = decode(st, q, moved, **kw)
    assert torch.equal(out, ref[0]) and torch.equal(lse, ref[1])


def test_chunks_with_more_pieces_than_a_record_holds_plan_nothing():
    """1024 sequences of at most 64 tokens on 16 cache heads: 32 chunks of about 2000 tokens, 30 pieces each,
    a record holds 20: such chunks are marked -1 and the workgroups cut for themselves."""
    dtype, B, Hc, G, D, P, ctx = torch.bfloat16, 1024, 16, 1, 64, 16, 128
    gen = torch.Generator().manual_seed(17)
    lens = torch.randint(0, 63, (B,), generator=gen).tolist()
    st = flat_state(92, B, Hc, D, P, ctx, dtype, lens=lens)
    q = randn(st.gen, (B, Hc * G, 1, D), dtype).to(DEV)
    pos = torch.tensor(lens, dtype=torch.int32, device=DEV)
    kw = dict(max_context=ctx, split_tokens=64)
    ref = decode(st, q, pos, **kw)
    plan = new_plan()
    decode(st, q, pos, phase="plan", plan=plan, **kw)
    rec = records(plan)
    n_chunks = 2 * torch.cuda.get_device_properties(0).multi_processor_count // Hc
    assert (rec[:n_chunks, 1] == B).all() and (rec[:n_chunks, 0] == -1).sum() >= n_chunks - 1
    got = decode(st, q, pos, plan=plan, **kw)
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    pk, pv = st.pool_planes()
    eo, el = O.decode_attention(f64(q), f64(pk), f64(pv), st.mirror.page_table, st.slots, np.array(lens), P)
    np.testing.assert_allclose(f64(got[0]), eo, atol=2e-2, rtol=1e-2)


def test_long_chunks_carry_more_page_ids_than_a_workgroup_has_threads():
    """8 sequences of 60 k to 100 k tokens on 16-token pages: 64 chunks of about 10 k tokens = 640 page ids,
    beyond the 256 a workgroup fetches with its record.  The pool is filled on the GPU; the planned launch
    against the unplanned one."""
    dtype, B, Hc, G, D, P, ctx = torch.bfloat16, 8, 8, 2, 64, 16, 100_000
    lens = [99_999, 60_000, 75_123, 88_001, 64_000, 91_777, 70_016, 83_333]
    st = PagedState(93, n_pages=sum(-(-(L + 1) // P) for L in lens) + 8, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype)
    for L in lens:
        st.add_sequence(L + 1)
    st.cache.kv_cache.normal_()
    q = randn(st.gen, (B, Hc * G, 1, D), dtype).to(DEV)
    k_new = randn(st.gen, (B, Hc, 1, D), dtype).to(DEV)
    v_new = randn(st.gen, (B, Hc, 1, D), dtype).to(DEV)
    pos = torch.tensor(lens, dtype=torch.int32, device=DEV)
    kw = dict(max_context=ctx, k_new=k_new, v_new=v_new)
    ref = decode(st, q, pos, **kw)
    pool = st.cache.kv_cache.clone()
    plan = new_plan()
    decode(st, q, pos, phase="plan", plan=plan, max_context=ctx)
    rec = records(plan)
    n = rec[0, 0]
    assert n >= 1 and rec[0, 1] == B
    last = rec[0, 4 + 6 * (n - 1):4 + 6 * n]
    assert last[5] + last[2] // P > 256  # page ids of chunk 0 beyond the first fetch
    got = decode(st, q, pos, plan=plan, **kw)
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    assert torch.equal(st.cache.kv_cache, pool)


def test_a_launch_without_an_even_cut_writes_no_plan_and_reads_none():
    """Three sequences: the launch goes split by split (or in one split); the plan call launches nothing and
    the buffer comes back as it went in."""
    dtype = torch.bfloat16
    st = PagedState(94, n_pages=96, page_size=32, max_batch=6, Hc=2, D=128, dtype=dtype)
    for L in (700, 64, 1300):
        st.add_sequence(L)
    st.prefill_random()
    q = randn(st.gen, (3, 4, 1, 128), dtype).to(DEV)
    pos = torch.tensor([699, 63, 1299], dtype=torch.int32, device=DEV)
    for kw in (dict(max_context=1408, split_tokens=256), dict(max_context=1408, split_tokens=2048)):
        plan = new_plan(0x5A)
        decode(st, q, pos, phase="plan", plan=plan, **kw)
        assert bool((plan == 0x5A).all())
        ref = decode(st, q, pos, **kw)
        got = decode(st, q, pos, plan=plan, **kw)
        assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])


def test_plan_arguments_are_checked():
    dtype = torch.bfloat16
    st = PagedState(95, n_pages=16, page_size=16, max_batch=4, Hc=1, D=64, dtype=dtype)
    st.add_sequence(40)
    st.prefill_random()
    q = randn(st.gen, (1, 1, 1, 64), dtype).to(DEV)
    pos = torch.tensor([39], dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="plan buffer needs"):
        decode(st, q, pos, max_context=64, plan=torch.zeros(1024, dtype=torch.uint8, device=DEV))
    with pytest.raises(RuntimeError, match="plan buffer needs"):
        decode(st, q, pos, max_context=64, phase="plan", plan=torch.zeros(1024, dtype=torch.uint8, device=DEV))
    with pytest.raises(RuntimeError, match="needs the plan tensor"):
        decode(st, q, pos, max_context=64, phase="plan")
    with pytest.raises(RuntimeError, match="uint8"):
        decode(st, q, pos, max_context=64, plan=torch.zeros(ops.decode_plan_bytes() // 4, dtype=torch.int32, device=DEV))


def test_plan_and_layers_replayed_from_one_graph_follow_the_positions():
    """What an engine captures: the plan, then the step's layers (here two, fused append), in one graph.  The
    positions advance in place between replays, so every replay plans anew; each replay against the eager,
    unplanned step on a copy of the pool."""
    dtype, B, Hc, G, D, P, split, ctx = torch.bfloat16, 72, 8, 2, 128, 32, 64, 512
    gen = torch.Generator().manual_seed(5)
    lens = torch.randint(0, ctx - 8, (B,), generator=gen).tolist()
    lens[0], lens[1] = ctx - 8, 0
    st = PagedState(96, n_pages=B * (ctx // P) + 8, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype, n_layers=2)
    for L in lens:
        st.add_sequence(min(L + 8, ctx))
    st.lens = lens
    st.prefill_random(layer=0)
    st.cache.kv_cache[1].copy_(st.cache.kv_cache[0].flip(-1))
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    pos = torch.tensor(lens, dtype=torch.int32, device=DEV)
    q = [randn(st.gen, (B, Hc * G, 1, D), dtype).to(DEV) for _ in range(2)]
    k_new = [randn(st.gen, (B, Hc, 1, D), dtype).to(DEV) for _ in range(2)]
    v_new = [randn(st.gen, (B, Hc, 1, D), dtype).to(DEV) for _ in range(2)]
    ws = torch.empty(ops.decode_workspace_bytes(B, Hc * G, D, ctx, split), dtype=torch.uint8, device=DEV)
    plan = new_plan()
    outs = [torch.empty(B, Hc * G, 1, D, dtype=dtype, device=DEV) for _ in range(2)]
    lses = [torch.empty(B, Hc * G, 1, dtype=torch.float32, device=DEV) for _ in range(2)]
    kw = dict(max_context=ctx, split_tokens=split)

    def layer(i, **extra):
        pk, pv = st.pool_planes(i)
        return ops.paged_decode(q[i], pk, pv, st.cache.page_table, bidx, pos, P, k_new=k_new[i], v_new=v_new[i], **kw, **extra)

    def step():
        ops.paged_decode(q[0], *st.pool_planes(0), st.cache.page_table, bidx, pos, P, phase="plan", plan=plan, **kw)
        for i in range(2):
            layer(i, workspace=ws, out=outs[i], lse=lses[i], plan=plan)

    pool = st.cache.kv_cache.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    st.cache.kv_cache.copy_(pool)
    for trial in range(4):
        for t in q + k_new + v_new:
            t.copy_(randn(st.gen, tuple(t.shape), dtype))
        before = st.cache.kv_cache.clone()
        g.replay()
        torch.cuda.synchronize()
        after = st.cache.kv_cache.clone()
        st.cache.kv_cache.copy_(before)
        for i in range(2):
            eo, el = layer(i)
            assert torch.equal(outs[i], eo) and torch.equal(lses[i], el), (trial, i)
        assert torch.equal(st.cache.kv_cache, after)
        pos += 1  # the next step of every sequence (the empty one gets its second token)


@pytest.mark.parametrize("fused", [True, False], ids=["append-fused", "append-first"])
def test_the_drop_in_plans_once_per_step_mask(monkeypatch, fused):
    """compiled_flex_attn_decode on a launch large enough for the even cut: the first layer that sees a step's
    mask writes the plan, the other layers of the step reuse it, the next step's mask plans anew; results
    equal the library call without a plan."""
    dtype, B, Hc, G, D, P, ctx, layers = torch.bfloat16, 64, 8, 2, 128, 64, 1024, 3
    gen = torch.Generator().manual_seed(9)
    lens = torch.randint(200, ctx - 4, (B,), generator=gen).tolist()
    st = PagedState(97, n_pages=B * (ctx // P) + 8, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype, n_layers=layers)
    for L in lens:
        st.add_sequence(min(L + 4, ctx))
    st.lens = lens
    st.cache.kv_cache.normal_()
    cache = st.cache
    cache.fuse_decode_append = fused
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    full = cache.create_causal_blockmask(B=B + 2, L=ctx)
    calls = []
    real = ops.paged_decode
    monkeypatch.setattr(ops, "paged_decode", lambda *a, **k: (calls.append(k.get("phase", "both")), real(*a, **k))[1])
    for step_no in range(2):
        pos = torch.tensor(lens, dtype=torch.int32, device=DEV) + step_no
        blk = pos // P
        logical = BlockMask.from_kv_blocks(
            full.kv_num_blocks[bidx, :, blk].view(B, 1, 1), full.kv_indices[bidx, :, blk].view(B, 1, 1, -1),
            full.full_kv_num_blocks[bidx, :, blk].view(B, 1, 1), full.full_kv_indices[bidx, :, blk].view(B, 1, 1, -1),
            BLOCK_SIZE=full.BLOCK_SIZE, mask_mod=lambda b, h, q, kv: q + pos[b] >= kv, seq_lengths=(1, ctx))
        mask = cache.convert_logical_block_mask(logical, bidx)
        _, split = cache.decode_launch(B, Hc * G, D, mask.max_context, Hc)
        calls.clear()
        for layer_id in range(layers):
            q = randn(st.gen, (B, Hc * G, 1, D), dtype).to(DEV)
            k = randn(st.gen, (B, Hc, 1, D), dtype).to(DEV)
            v = randn(st.gen, (B, Hc, 1, D), dtype).to(DEV)
            before = cache.kv_cache[layer_id].clone()
            K, V = cache.insert_kv(layer_id, k, v, input_pos=pos.view(B, 1), batch_idx=bidx)
            out, aux = A.compiled_flex_attn_decode(q, K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
            after = cache.kv_cache[layer_id].clone()  # (reading kv_cache writes any deferred append first)
            if fused:  # the reference step appends in its launch as well
                cache.kv_cache[layer_id].copy_(before)
            fresh = dict(k_new=k, v_new=v) if fused else {}
            eo, el = real(q, cache.kv_cache[layer_id, 0, 0], cache.kv_cache[layer_id, 1, 0], cache.page_table, bidx, pos,
                          P, mask.max_context, split_tokens=split, **fresh)
            assert torch.equal(out, eo) and torch.equal(aux.lse.view(el.shape), el), (step_no, layer_id)
            assert torch.equal(cache.kv_cache[layer_id], after)
        assert calls.count("plan") == 1 and calls[0] == "plan", calls
    rec = records(cache.decode_plan())
    assert rec[0, 0] >= 1 and rec[0, 1] == B  # the launch was large enough to be cut evenly: the plan was read
