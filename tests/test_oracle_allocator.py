"""Pins oracle.PagedAllocator (restating reference paged_attention.py:39-182).

Known answers are traced by hand from the reference source and stored in
tests/golden/allocator_kat.json; the invariants are what any correct page
allocator must keep.
"""

import json
import os
import random

import numpy as np
import pytest

from oracle.paged_kv_oracle import PagedAllocator

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "allocator_kat.json")


def run_trace(alloc, trace):
    out = []
    for op in trace:
        name = op[0]
        if name == "allocate":
            out.append(alloc.allocate())
        elif name == "reserve":
            out.append(alloc.reserve(op[1], op[2]))
        elif name == "erase":
            alloc.erase(op[1])
            out.append(None)
        elif name == "can_reserve":
            out.append(alloc.can_reserve(op[1], op[2] if len(op) > 2 else None))
    return out


def test_fresh_state():
    a = PagedAllocator(n_pages=8, page_size=4, max_batch_size=4)
    assert a.free_pages == [7, 6, 5, 4, 3, 2, 1]  # page 0 reserved, stack top = 1
    assert a.free_batch_idx == [3, 2, 1]  # slot 0 reserved
    assert (a.page_table[0] == 0).all() and (a.page_table[1:] == -1).all()
    assert (a.physical_to_logical == -1).all()
    assert a.capacity == [0, 0, 0, 0]


@pytest.mark.parametrize("case", json.load(open(GOLDEN))["cases"], ids=lambda c: c["name"])
def test_known_answers(case):
    a = PagedAllocator(**case["init"])
    got = run_trace(a, case["trace"])
    assert got == case["returns"]
    exp = case["final"]
    assert a.free_pages == exp["free_pages"]
    assert a.free_batch_idx == exp["free_batch_idx"]
    assert a.capacity == exp["capacity"]
    assert a.page_table_cpu == exp["page_table_cpu"]
    assert a.page_table.tolist() == exp["page_table"]
    assert a.physical_to_logical.tolist() == exp["physical_to_logical"]


def test_reserve_failure_message_and_dry_run():
    a = PagedAllocator(n_pages=4, page_size=4, max_batch_size=3)
    b = a.allocate()
    assert a.can_reserve(12) and not a.can_reserve(13)
    assert a.reserve(b, 13, dry_run=True) is False
    with pytest.raises(RuntimeError) as e:
        a.reserve(b, 13)
    assert str(e.value) == (
        "Cannot reserve 4 pages for a sequence of length 13 in batch 1. "
        "Only 3 pages available. Current capacity is 0 tokens."
    )
    # the failed call changed nothing
    assert a.free_pages == [3, 2, 1] and a.capacity[b] == 0 and (a.page_table[b] == -1).all()
    assert a.reserve(b, 12) and a.num_free_pages == 0
    assert a.reserve(b, 5) is True  # already covered: no-op
    assert not a.can_reserve(1)  # no pages left


def check_invariants(a, live):
    P, Np = a.page_size, a.n_pages
    owned = [p for b in live for p in a.page_table_cpu[b]]
    assert len(owned) == len(set(owned)), "a page is mapped twice"
    assert 0 not in owned and 0 not in a.free_pages, "page 0 must never be handed out"
    assert sorted(owned + a.free_pages) == list(range(1, Np))
    assert sorted(live + a.free_batch_idx) == list(range(1, a.max_batch_size))
    for b in live:
        pages = a.page_table_cpu[b]
        assert a.capacity[b] == P * len(pages)
        assert a.page_table[b, :len(pages)].tolist() == pages
        assert (a.page_table[b, len(pages):] == -1).all()
        for lb, p in enumerate(pages):
            assert a.physical_to_logical[b, p] == lb
        assert (a.physical_to_logical[b] >= 0).sum() == len(pages)
    for b in a.free_batch_idx:
        assert a.capacity[b] == 0 and a.page_table_cpu[b] == []
    assert (a.page_table[0] == 0).all()


@pytest.mark.parametrize("seed", range(5))
def test_random_trace_invariants(seed):
    rng = random.Random(seed)
    a = PagedAllocator(n_pages=33, page_size=8, max_batch_size=9)
    live, want = [], {}
    for _ in range(400):
        r = rng.random()
        if r < 0.25 and a.free_batch_idx and a.can_reserve(1):
            b = a.allocate()
            live.append(b)
            want[b] = 0
        elif r < 0.75 and live:
            b = rng.choice(live)
            n = want[b] + rng.randint(1, 20)
            if a.can_reserve(n, b):
                a.reserve(b, n)
                want[b] = n
                assert a.capacity[b] >= n and a.capacity[b] - n < a.page_size
            else:
                with pytest.raises(RuntimeError):
                    a.reserve(b, n)
        elif live:
            b = live.pop(rng.randrange(len(live)))
            a.erase(b)
            del want[b]
        check_invariants(a, live)
