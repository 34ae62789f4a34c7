"""Host-side checks that need no GPU: the C-ABI library loads and exports what the
header declares, the Python mirror keeps the reference's allocator semantics and
mask structure, and nothing silently falls back to a CPU path."""

import json
import os
import random
import re
import sys

import numpy as np
import pytest
import torch
from torch.nn.attention.flex_attention import create_block_mask

import falcon_perception_amd as fpa
from falcon_perception_amd import _native
from falcon_perception_amd import attention as A
from falcon_perception_amd.paged_attention import PagedKVCache
from oracle import paged_kv_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, "include", "fp_paged_kv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fp_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(native_lib):
    names = header_functions()
    assert len(names) >= 9
    for n in names:
        assert hasattr(native_lib, n), f"{n} declared in the header but not exported"
    assert sorted(_native.SIGNATURES) == names
    assert native_lib.fp_abi_version() == _native.FP_ABI_VERSION


def header_declarations():
    """name -> number of parameters, from the C declarations of the header."""
    text = open(os.path.join(ROOT, "include", "fp_paged_kv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    decls = {}
    for name, params in re.findall(r"\b(fp_[a-z0-9_]+)\s*\(([^()]*)\)\s*;", text):
        params = params.strip()
        decls[name] = 0 if params in ("", "void") else params.count(",") + 1
    return decls


def test_ctypes_signatures_have_the_arity_of_the_header():
    decls = header_declarations()
    assert sorted(decls) == header_functions()
    for name, n in decls.items():
        restype, argtypes = _native.SIGNATURES[name]
        assert len(argtypes) == n, f"{name}: header declares {n} parameters, the binding passes {len(argtypes)}"


def test_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 and as C++ with nothing but the standard headers."""
    import shutil
    import subprocess

    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    names = header_functions()
    src = tmp_path / "use_header.c"
    table = ", ".join(f"(void (*)(void)){n}" for n in names)
    src.write_text('#include "fp_paged_kv.h"\nvoid (*const fp_table[])(void) = {' + table + "};\n")
    inc = os.path.join(ROOT, "include")
    for cmd in (["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror"], ["g++", "-x", "c++", "-std=c++11", "-Wall", "-Werror"]):
        res = subprocess.run(cmd + ["-I", inc, "-fsyntax-only", str(src)], capture_output=True, text=True)
        assert res.returncode == 0, res.stderr


def test_argument_errors_come_back_as_codes_not_crashes(native_lib):
    # no device work: every call below is rejected by the host-side checks
    assert native_lib.fp_paged_decode_workspace_bytes(4, 8, 128, 1024, 100) < 0  # split not a multiple of 64
    assert b"multiple of 64" in native_lib.fp_last_error()
    assert native_lib.fp_paged_decode_workspace_bytes(4, 8, 128, 1024, 256) == 4 * 8 * 4 * 130 * 4
    assert native_lib.fp_paged_decode_workspace_bytes(4, 8, 128, 256, 256) == 0  # one split: no workspace
    assert native_lib.fp_paged_decode_default_split(64, 8, 4096, 128) % 64 == 0
    rc = native_lib.fp_kv_append(None, None, None, None, 0, 0, 0, 0, 0, 0, None, 0, None, None, 0,
                                 4, 2, 1, 8, 4, 8, 4, 32, 7, 1, None)
    assert rc == -2 and b"dtype" in native_lib.fp_last_error()
    rc = native_lib.fp_kv_append(None, None, None, None, 0, 0, 0, 0, 0, 0, None, 0, None, None, 0,
                                 4, 2, 1, 8, 4, 8, 4, 32, 1, 1, None)
    assert rc == -1 and b"null" in native_lib.fp_last_error()


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", "/nonexistent/libfp_paged_kv.so")
    with pytest.raises(RuntimeError, match="no other compute path"):
        _native.lib()


def test_no_cpu_fallback():
    c = PagedKVCache(8, 4, 4, 2, 8, 1, torch.float32, device="cpu")
    b = c.allocate()
    c.reserve(b, torch.tensor([b]), 4)
    k = torch.zeros(1, 2, 1, 8)
    with pytest.raises(RuntimeError, match="GPU only"):
        c.insert_kv(0, k, k, input_pos=torch.zeros(1, 1, dtype=torch.int32), batch_idx=torch.tensor([b]))


def snapshot(c):
    return (list(c.free_pages), list(c.free_batch_idx), list(c.capacity),
            [list(x) for x in c.page_table_cpu], c.page_table.tolist(), c.physical_to_logical.tolist())


def o_snapshot(a):
    return (list(a.free_pages), list(a.free_batch_idx), list(a.capacity),
            [list(x) for x in a.page_table_cpu], a.page_table.tolist(), a.physical_to_logical.tolist())


def test_allocator_known_answers():
    cases = json.load(open(os.path.join(ROOT, "tests", "golden", "allocator_kat.json")))["cases"]
    for case in cases:
        i = case["init"]
        c = PagedKVCache(i["n_pages"], i["page_size"], i["max_batch_size"], 1, 4, 1, torch.float32, device="cpu")
        got = []
        for op in case["trace"]:
            if op[0] == "allocate":
                got.append(c.allocate())
            elif op[0] == "reserve":
                got.append(c.reserve(op[1], torch.tensor([op[1]]), op[2]))
            elif op[0] == "erase":
                c.erase(op[1])
                got.append(None)
            else:
                got.append(c.can_reserve(op[1], op[2] if len(op) > 2 else None))
        assert got == case["returns"], case["name"]
        f = case["final"]
        assert snapshot(c) == (f["free_pages"], f["free_batch_idx"], f["capacity"], f["page_table_cpu"],
                               f["page_table"], f["physical_to_logical"]), case["name"]


@pytest.mark.parametrize("seed", range(3))
def test_allocator_follows_the_oracle_on_random_traces(seed):
    rng = random.Random(seed)
    c = PagedKVCache(33, 8, 9, 1, 4, 1, torch.float32, device="cpu")
    a = O.PagedAllocator(33, 8, 9)
    assert c.kv_cache.shape == (1, 2, 1, 1, 33 * 8, 4) and c.kv_shape == tuple(c.kv_cache.shape)
    live, want = [], {}
    for _ in range(300):
        r = rng.random()
        if r < 0.25 and c.free_batch_idx and c.can_reserve(1):
            b = c.allocate()
            assert b == a.allocate()
            live.append(b)
            want[b] = 0
        elif r < 0.75 and live:
            b = rng.choice(live)
            n = want[b] + rng.randint(1, 20)
            assert c.can_reserve(n, b) == a.can_reserve(n, b)
            if c.can_reserve(n, b):
                c.reserve(b, torch.tensor([b]), n)
                a.reserve(b, n)
                want[b] = n
            else:
                with pytest.raises(RuntimeError) as e1:
                    c.reserve(b, torch.tensor([b]), n)
                with pytest.raises(RuntimeError) as e2:
                    a.reserve(b, n)
                assert str(e1.value) == str(e2.value)
        elif live:
            b = live.pop(rng.randrange(len(live)))
            c.erase(b)
            a.erase(b)
            del want[b]
        assert snapshot(c) == o_snapshot(a)
        assert c.num_free_pages == a.num_free_pages


@pytest.mark.parametrize("n_blocks", [1, 3, 8])
def test_causal_blockmask_equals_torch_create_block_mask(n_blocks):
    P, B = 4, 3
    c = PagedKVCache(16, P, 4, 1, 4, 1, torch.float32, device="cpu")
    L = n_blocks * P
    got = c.create_causal_blockmask(B, L)
    ref = create_block_mask(A.get_causal_mask_mod(), B, None, L, L, device="cpu", BLOCK_SIZE=P)
    assert got.BLOCK_SIZE == ref.BLOCK_SIZE and got.seq_lengths == ref.seq_lengths
    assert got.kv_indices.shape == ref.kv_indices.shape and got.kv_indices.dtype == ref.kv_indices.dtype
    assert torch.equal(got.kv_num_blocks, ref.kv_num_blocks)
    assert torch.equal(got.kv_indices, ref.kv_indices)
    if n_blocks > 1:
        assert torch.equal(got.full_kv_num_blocks, ref.full_kv_num_blocks)
        assert torch.equal(got.full_kv_indices, ref.full_kv_indices)
    assert torch.equal(got.to_dense(), ref.to_dense())
    # the engine slices it like this (reference paged_inference.py:803-826)
    bidx = torch.tensor([2, 1])
    blk = torch.tensor([0, n_blocks - 1])
    assert got.kv_num_blocks[bidx, :, blk].shape == (2, 1)
    assert got.kv_indices[bidx, :, blk].view(2, 1, 1, -1).shape == (2, 1, 1, n_blocks)


def test_convert_rejects_a_foreign_block_size():
    c = PagedKVCache(16, 4, 4, 1, 4, 1, torch.float32, device="cpu")
    other = PagedKVCache(16, 8, 4, 1, 4, 1, torch.float32, device="cpu").create_causal_blockmask(2, 16)
    with pytest.raises(RuntimeError, match="same column block size"):
        c.convert_logical_block_mask(other)


def test_physical_mask_mod_matches_the_oracle():
    c = PagedKVCache(10, 4, 4, 1, 4, 1, torch.float32, device="cpu")
    c.free_pages = [3, 8, 1, 6, 9, 2, 7, 5, 4]
    slots = []
    for L in (6, 9):
        b = c.allocate()
        c.reserve(b, torch.tensor([b]), L)
        slots.append(b)
    bidx = torch.tensor(slots)
    mod = c.get_mask_mod(A.get_causal_mask_mod(), bidx)
    p2l = c.physical_to_logical.numpy()
    for b in range(2):
        for q in (0, 5):
            phys = torch.arange(40)
            got = mod(torch.tensor(b), torch.tensor(0), torch.tensor(q), phys)
            exp = [O.physical_mask(p2l, slots, 4, lambda _b, qq, kv: qq >= kv, b, q, int(p)) for p in phys]
            assert got.tolist() == exp


def test_mask_mod_factories_match_the_oracle_tables():
    from tests.test_oracle_masks import EOI, SOI, packed_case

    ids, bidx, pos, spans = packed_case([(1, [("t", 2), ("i", 5), ("t", 3)]), (2, [("i", 3), ("t", 2)])])
    t_ids = torch.from_numpy(ids)[None]
    mod = A.get_image_prefix_mask_mod(t_ids, SOI, EOI)
    L = len(ids)
    qq, kk = torch.meshgrid(torch.arange(L), torch.arange(L), indexing="ij")
    got = mod(torch.tensor(0), torch.tensor(0), qq, kk).numpy()
    img, idx = O.image_prefix_tables(ids, SOI, EOI)
    exp = img[:, None] & img[None, :] & (idx[:, None] == idx[None, :])
    assert np.array_equal(got, exp)
    assert A.offset_mask_mod(A.get_causal_mask_mod(), 3)(0, 0, torch.tensor(1), torch.tensor(4)).item()


@pytest.fixture(autouse=True)
def restore_install_defaults(monkeypatch):
    """`install()` writes class-wide defaults; every test starts from the bare ones and leaves them so."""
    monkeypatch.setattr(PagedKVCache, "default_kv_rep", 1)
    monkeypatch.setattr(PagedKVCache, "default_qk_normalised", False)
    monkeypatch.setattr(PagedKVCache, "default_fuse_decode_append", False)


def test_install_serves_the_reference_module_names():
    saved = {k: sys.modules.get(k) for k in
             ("falcon_perception.kv_cache", "falcon_perception.paged_attention", "falcon_perception.attention")}
    try:
        fpa.install()
        assert sys.modules["falcon_perception.paged_attention"].PagedKVCache is PagedKVCache
        assert sys.modules["falcon_perception.attention"].compiled_flex_attn_decode is A.compiled_flex_attn_decode
        assert sys.modules["falcon_perception.kv_cache"].KVCacheBase is fpa.KVCacheBase
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v


def test_sparse_page_table_allocator():
    """max_blocks_per_seq: same allocator decisions as the dense table (free lists, capacities, the
    mapped prefix of every row), a narrower table, no inverse table, and a per-sequence length limit."""
    dense = PagedKVCache(40, 4, 5, 1, 4, 1, torch.float32, device="cpu")
    sparse = PagedKVCache(40, 4, 5, 1, 4, 1, torch.float32, device="cpu", max_blocks_per_seq=6)
    assert sparse.page_table.shape == (5, 6) and sparse.physical_to_logical is None
    assert sparse.page_table[0].tolist() == [0] * 6  # the reserved row still points at page 0
    for c in (dense, sparse):
        a, b = c.allocate(), c.allocate()
        c.reserve(a, None, 9)
        c.reserve(b, None, 24)
        c.reserve(a, None, 13)
        c.erase(b)
        b2 = c.allocate()
        c.reserve(b2, None, 5)
    assert sparse.free_pages == dense.free_pages and sparse.capacity == dense.capacity
    assert sparse.page_table_cpu == dense.page_table_cpu
    assert sparse.page_table.tolist() == dense.page_table[:, :6].tolist()
    assert int(sparse.page_table.max()) >= 6  # page ids are not bounded by the table width
    assert sparse.can_reserve(24, 1) is True and sparse.can_reserve(25, 1) is False and dense.can_reserve(25, 1) is True
    with pytest.raises(RuntimeError, match="6 blocks"):
        sparse.reserve(1, None, 25)
    with pytest.raises(ValueError):
        PagedKVCache(8, 4, 2, 1, 4, 1, torch.float32, device="cpu", max_blocks_per_seq=9)


def test_prefill_row_limit_survives_inference_mode():
    """The reference's engine builds input_pos inside torch.inference_mode() (paged_inference.py:646-675,
    1331); such tensors have no version counter.  The row limits are recomputed when a new step starts
    (layer id not growing) or another positions tensor arrives."""
    c = PagedKVCache(8, 4, 4, 2, 8, 1, torch.float32, device="cpu")
    row_hi = torch.tensor([1, 5, 5, 5, 5, 6], dtype=torch.int32)
    with torch.inference_mode():
        bidx = torch.ones(1, 6, dtype=torch.int64)
        m = A.HybridPrefillMask(c, bidx, torch.zeros(1, 6, dtype=torch.int64), 1, 2, 128, row_hi=row_hi)
        pos = torch.arange(10, 16)[None]
        with pytest.raises(RuntimeError):
            pos._version  # what the key must not touch
        lim0 = m.row_limit(pos, 0)
        assert lim0.tolist() == [11, 15, 15, 15, 15, 16]
        assert m.row_limit(pos, 1) is lim0  # later layers of the step reuse it
        pos.add_(100)  # the engine's next step may reuse the buffer
        assert m.row_limit(pos, 0).tolist() == [111, 115, 115, 115, 115, 116]
        assert m.row_limit(torch.arange(6)[None], 1).tolist() == [1, 5, 5, 5, 5, 6]


def test_install_serves_the_reference_module_names_and_sets_kv_rep(monkeypatch):
    monkeypatch.setattr(PagedKVCache, "default_kv_rep", 1)
    for name in ("falcon_perception.kv_cache", "falcon_perception.paged_attention", "falcon_perception.attention"):
        monkeypatch.delitem(sys.modules, name, raising=False)
    fpa.install(kv_rep=2)
    import importlib

    assert importlib.import_module("falcon_perception.paged_attention").PagedKVCache is PagedKVCache
    assert importlib.import_module("falcon_perception.attention").compiled_flex_attn_decode is A.compiled_flex_attn_decode
    # what the engine builds (paged_inference.py:321-330): n_heads cached heads; the cache now knows the V copies
    c = PagedKVCache(8, 4, 4, 16, 8, 1, torch.float32, device="cpu")
    assert c.kv_rep == 2 and c.v_copies_are_identical()
    c.kv_cache[0, 1, 0, 1, 5] = 1.0  # head 1 no longer equals head 0
    assert not c.v_copies_are_identical()
    assert PagedKVCache(8, 4, 4, 3, 8, 1, torch.float32, device="cpu").kv_rep == 1  # 3 heads: no groups of 2
    with pytest.raises(ValueError):
        fpa.install(kv_rep=0)
    # the constructor's own argument wins over the class default and is validated
    assert PagedKVCache(8, 4, 4, 16, 8, 1, torch.float32, device="cpu", kv_rep=1).kv_rep == 1
    with pytest.raises(ValueError):
        PagedKVCache(8, 4, 4, 16, 8, 1, torch.float32, device="cpu", kv_rep=3)


def test_install_sets_what_an_unedited_engine_cannot_say(monkeypatch):
    for attr in ("default_kv_rep", "default_qk_normalised", "default_fuse_decode_append"):
        monkeypatch.setattr(PagedKVCache, attr, getattr(PagedKVCache, attr))
    for name in ("falcon_perception.kv_cache", "falcon_perception.paged_attention", "falcon_perception.attention"):
        monkeypatch.delitem(sys.modules, name, raising=False)
    bare = PagedKVCache(8, 4, 4, 16, 8, 1, torch.float32, device="cpu")
    assert not bare.fuse_decode_append and not bare.qk_normalised and bare.score_bound(64, None) == 0.0
    fpa.install(kv_rep=2, qk_norm=True)
    c = PagedKVCache(8, 4, 4, 16, 64, 1, torch.float32, device="cpu")
    assert c.fuse_decode_append and c.qk_normalised and c.kv_rep == 2
    assert c.score_bound(64, None) == pytest.approx(1.1 * 8.0) and c.score_bound(64, 0.25) == pytest.approx(1.1 * 16.0)
    fpa.install(fuse_decode_append=False)
    c = PagedKVCache(8, 4, 4, 16, 64, 1, torch.float32, device="cpu")
    assert not c.fuse_decode_append and not c.qk_normalised and c.kv_rep == 1


def test_reserve_beyond_the_pool_raises_the_reference_message_on_a_dense_table():
    """`paged_attention.py:138-143`: the message names the pages asked for and the pages left.  With the dense
    table the pool always runs out before the table does; only a sparse table has a message of its own."""
    c = PagedKVCache(8, 4, 4, 2, 8, 1, torch.float32, device="cpu")
    b = c.allocate()
    with pytest.raises(RuntimeError) as e:
        c.reserve(b, None, 9 * 4)
    assert str(e.value) == ("Cannot reserve 9 pages for a sequence of length 36 in batch 1. "
                            "Only 7 pages available. Current capacity is 0 tokens.")
    assert c.reserve(b, None, 9 * 4, dry_run=True) is False
    sparse = PagedKVCache(64, 4, 4, 2, 8, 1, torch.float32, device="cpu", max_blocks_per_seq=3)
    b = sparse.allocate()
    with pytest.raises(RuntimeError, match="the page table holds 3 blocks"):
        sparse.reserve(b, None, 16)
    assert sparse.reserve(b, None, 16, dry_run=True) is False and sparse.reserve(b, None, 12, dry_run=True) is True


def test_bench_reads_traffic_from_the_profiles_and_refuses_several_gpus():
    import subprocess

    import bench

    # the decode workloads share one summary (a line per workload), the other kernels have a file each
    for wl in ("cfg1", "cfg2", "cfg2x", "cfg2xs", "cfg2d64", "cfg2f32", "cfg4d", "cfg5"):
        t = bench.profiled_traffic("paged_decode", wl)
        assert t is not None and t > 1e6, wl
    for kernel in ("kv_append", "kv_gather", "qkv_rope_append"):
        assert bench.profiled_traffic(kernel, "32768x16") > 2.6e8
    assert bench.profiled_traffic("paged_decode", "no_such_workload") is None
    # traffic must not fall below the algorithmic bytes it is compared with (cfg2: 666.07 MB)
    assert 666.0e6 < bench.profiled_traffic("paged_decode", "cfg2") < 1.05 * 666.1e6
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode == 2 and "ONE GPU" in res.stderr and not res.stdout.strip()


def test_noalloc_entry_point_rejects_what_its_array_cannot_hold(native_lib):
    # host-side checks only: nothing below reaches the GPU
    args = lambda B, split: (None, 0, 0, None, None, None, 0, None, None, 0, None, 0, 0, None, None,
                             B, 32, 32, 1, 128, 16, 512, 4, 128, 8192, split, 1.0, 1, None)
    rc = native_lib.fp_paged_decode_noalloc(*args(4096, 64))
    assert rc == -4 and b"the library's array holds" in native_lib.fp_last_error()
    assert native_lib.fp_paged_decode_workspace_bytes(4096, 32, 128, 8192, 64) > _native.NOALLOC_SCRATCH_BYTES
    assert native_lib.fp_paged_decode_noalloc(*args(-1, 64)) == -1
    assert native_lib.fp_paged_decode_noalloc(*args(4, 100)) == -1 and b"multiple of 64" in native_lib.fp_last_error()
    # the header's limit and the Python mirror agree
    text = open(os.path.join(ROOT, "include", "fp_paged_kv.h")).read()
    assert re.search(r"#define FP_NOALLOC_SCRATCH_BYTES \(64ll << 20\)", text) and _native.NOALLOC_SCRATCH_BYTES == 64 << 20


def test_hybrid_row_limits_argument_errors(native_lib):
    assert native_lib.fp_hybrid_row_limits(None, None, None, 0, -1, 1, 2, None, None, None) == -1
    assert native_lib.fp_hybrid_row_limits(None, None, None, 0, 70000, 1, 2, None, None, None) == -2
    assert native_lib.fp_hybrid_row_limits(None, None, None, 0, 0, 1, 2, None, None, None) == 0  # an empty row is fine
    assert native_lib.fp_hybrid_row_limits(None, None, None, 0, 5, 1, 2, None, None, None) == -1  # null pointers


def test_only_the_documented_kernels_use_scratch_memory():
    """A kernel whose registers spill to scratch memory cannot be launched for the first time while a stream
    is being captured into a graph (the runtime sets the memory up at that launch).  The header promises that
    this concerns nothing but the four-wavefront instances of the 16-bit prefill kernel at head_dim 64; the
    compiler's own report of every kernel of the last build is held against that promise."""
    import importlib.util
    import re

    spec = importlib.util.spec_from_file_location("fp_build_native", os.path.join(ROOT, "falcon-perception_amd", "build_native.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    usage = mod.resource_usage()
    assert len(usage) > 300  # every template instance of the nine sources
    for family in ("paged_decode_kernel", "paged_decode_merge", "kv_append_kernel", "kv_gather_kernel", "qkv_rope",
                   "hybrid_row_limits_kernel", "convert_block_ids_kernel", "paged_prefill_kernel", "paged_prefill_f32_kernel",
                   "paged_prefill_merge_kernel", "probe_kernel"):
        assert any(family in name for name in usage), family
    # paged_prefill_kernel<E, 64, G, pow2, 4 wavefronts, bounded>
    allowed = re.compile(r"paged_prefill_kernelINS_\d?(BF16|F16)ELi64ELi\dELb[01]ELi4ELb[01]E")
    spilling = {name: u["scratch"] for name, u in usage.items() if u["scratch"] > 0}
    assert spilling, "the header's exception list can go: no kernel uses scratch any more"
    for name, scratch in spilling.items():
        assert allowed.search(name), f"{name} spills {scratch} bytes per lane and may be launched under graph capture"
        assert scratch <= 64
