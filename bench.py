#!/usr/bin/env python3
"""Benchmark of the paged KV-cache hot path on one MI355X.

A step is one layer of one decode step at the serving shape of BASELINE.json
configs[1]: append one new K/V row per sequence into the page pool, then
single-query paged attention over every cached row (split-K + merge).  Inputs are
synthetic, seeded, and resident in HBM before the timed region starts.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2]

Prints ONE JSON line: whole-job algorithmic HBM throughput (`value`, GB/s) with
the decode kernel's roofline and a CPU baseline timed on the host cores.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time
from dataclasses import dataclass, field

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "falcon-perception_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import torch  # noqa: E402

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published peak
MFMA_F32_PEAK_TFLOPS = 157.3    # MI355X dense fp32 MFMA, published peak
MODEL_LAYERS = 28       # Falcon Perception 0.6B (reference __init__.py:36)

# name -> shape of the decode workloads of BASELINE.json (configs[0], [1], [3] decode part, [4])
DECODE_WORKLOADS = {
    "cfg1": dict(seed=1, dtype="f32", B=4, Hq=8, Hc=8, D=64, P=64, n_pages=64, prefix=0, lo=64, hi=512),
    "cfg2": dict(seed=2, dtype="bf16", B=64, Hq=16, Hc=8, D=128, P=128, n_pages=4096, prefix=1024, lo=64, hi=3072),
    "cfg2x": dict(seed=2, dtype="bf16", B=64, Hq=16, Hc=16, D=128, P=128, n_pages=4096, prefix=1024, lo=64, hi=3072),
    # the same expanded cache read as what it is: K per query head, V in groups of 2 identical copies
    "cfg2xs": dict(seed=2, dtype="bf16", B=64, Hq=16, Hc=16, D=128, P=128, n_pages=4096, prefix=1024, lo=64, hi=3072,
                   kv_rep=2),
    "cfg4d": dict(seed=4, dtype="bf16", B=32, Hq=16, Hc=8, D=128, P=64, n_pages=8192, prefix=0, lo=512, hi=8192),
    "cfg5": dict(seed=5, dtype="bf16", B=256, Hq=32, Hc=8, D=128, P=128, n_pages=None, prefix=4096, lo=256, hi=12288),
    # cfg2 at the head_dim of the reference's OCR and 300M variants (reference __init__.py:78-85)
    "cfg2d64": dict(seed=2, dtype="bf16", B=64, Hq=16, Hc=8, D=64, P=128, n_pages=4096, prefix=1024, lo=64, hi=3072),
    # cfg2 in the reference's default dtype (reference server/config.py:38)
    "cfg2f32": dict(seed=2, dtype="f32", B=64, Hq=16, Hc=8, D=128, P=128, n_pages=4096, prefix=1024, lo=64, hi=3072),
}
DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
# token ids of the synthetic packed rows (any five distinct values): start / end of an image block, a token
# inside it, a text token, padding.  A span is [soi, eoi): the soi row is inside, the eoi row is not
# (reference attention.py:77-79), and the text follows (data.py:513-522).
SOI_ID, EOI_ID, IMG_ID, TXT_ID, PAD_ID = 3, 4, 7, 11, 0



def profiled_traffic(kernel: str, workload: str) -> float | None:
    """HBM bytes per launch of `kernel` at `workload` as a rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE pair
    measured them (each scaled by the same counter on a plain copy of known size): the line
    `traffic_bytes_per_launch = N` of profiles/<kernel>_<workload>_hbm_traffic.md, or the line
    `traffic_bytes_per_launch[<workload>] = N` of profiles/<kernel>_hbm_traffic.md; None when no such
    summary has been recorded."""
    import re

    for name, pattern in ((f"{kernel}_{workload}_hbm_traffic.md", r"traffic_bytes_per_launch\s*=\s*([0-9.eE+]+)"),
                          (f"{kernel}_hbm_traffic.md",
                           r"traffic_bytes_per_launch\[" + re.escape(workload) + r"\]\s*=\s*([0-9.eE+]+)")):
        try:
            m = re.search(pattern, open(os.path.join(ROOT, "profiles", name)).read())
        except OSError:
            continue
        if m:
            return float(m.group(1))
    return None


@dataclass
class DecodeCase:
    """One decode step's operands, all on the device."""

    name: str
    cfg: dict
    cache: object
    lens: list            # context length of each sequence before the step
    batch_idx: torch.Tensor
    input_pos: torch.Tensor   # [B] int32 position of the new token (= lens)
    q: torch.Tensor
    k_new: torch.Tensor
    v_new: torch.Tensor
    max_context: int
    split_tokens: int = 0
    workspace: torch.Tensor | None = None
    out: torch.Tensor | None = None
    lse: torch.Tensor | None = None
    plan: torch.Tensor | None = None  # the step's plan (fp_paged_decode_plan), read by the launches while `planned`
    planned: bool = True
    layer_steps: int = 0              # layer-steps run through `run_step` so far
    extra: dict = field(default_factory=dict)

    @property
    def page_size(self):
        return self.cache.page_size

    @property
    def page_table(self):
        return self.cache.page_table

    @property
    def _plan(self):
        return self.plan if self.planned else None

    def make_plan(self):
        """What a model does once per decode step, before its first layer: positions, slots and page table
        are those of every layer of the step."""
        from falcon_perception_amd import ops

        ops.paged_decode(self.q, self.pool_k, self.pool_v, self.cache.page_table, self.batch_idx, self.input_pos,
                         self.page_size, self.max_context, split_tokens=self.split_tokens, phase="plan",
                         plan=self.plan, kv_rep=self.cfg.get("kv_rep", 1))

    def run_step(self):
        """The layer-step at the rate a model of MODEL_LAYERS layers runs it: the plan of the step is written
        before every MODEL_LAYERS-th layer-step (inside whatever region is being timed), and the fused
        append + decode launches read it."""
        if self.planned and self.layer_steps % MODEL_LAYERS == 0:
            self.make_plan()
        self.layer_steps += 1
        return self.run_fused()

    @property
    def pool_k(self):
        return self.cache.kv_cache[0, 0, 0]

    @property
    def pool_v(self):
        return self.cache.kv_cache[0, 1, 0]

    def append(self):
        from falcon_perception_amd import ops

        ops.kv_append(self.pool_k, self.pool_v, self.k_new, self.v_new, self.cache.page_table,
                      self.batch_idx, self.input_pos.view(-1, 1), self.page_size, clamp_negative=True)

    def attend(self, phase="both"):
        from falcon_perception_amd import ops

        return ops.paged_decode(self.q, self.pool_k, self.pool_v, self.cache.page_table, self.batch_idx,
                                self.input_pos, self.page_size, self.max_context,
                                split_tokens=self.split_tokens, workspace=self.workspace,
                                out=self.out, lse=self.lse, phase=phase, kv_rep=self.cfg.get("kv_rep", 1),
                                plan=self._plan)

    def run(self):
        self.append()
        return self.attend()

    def run_fused(self):
        """The same step as one library call: the new rows are appended by the decode kernel itself."""
        from falcon_perception_amd import ops

        return ops.paged_decode(self.q, self.pool_k, self.pool_v, self.cache.page_table, self.batch_idx,
                                self.input_pos, self.page_size, self.max_context,
                                split_tokens=self.split_tokens, workspace=self.workspace,
                                out=self.out, lse=self.lse, k_new=self.k_new, v_new=self.v_new,
                                kv_rep=self.cfg.get("kv_rep", 1), plan=self._plan)

    def run_fused_gated(self):
        """run_fused plus the caller's post-attention sink gate (reference model.py:122-127) inside the
        merge pass, written in the [B, 1, Hq * D] layout of the output projection."""
        from falcon_perception_amd import ops

        c = self.cfg
        if "sinks" not in self.extra:
            self.extra["sinks"] = torch.linspace(-2.0, 2.0, c["Hq"], device=self.q.device)
            self.extra["flat"] = torch.empty((c["B"], 1, c["Hq"] * c["D"]), dtype=self.q.dtype, device=self.q.device)
        out = self.extra["flat"].view(c["B"], 1, c["Hq"], c["D"]).permute(0, 2, 1, 3)
        return ops.paged_decode(self.q, self.pool_k, self.pool_v, self.cache.page_table, self.batch_idx,
                                self.input_pos, self.page_size, self.max_context,
                                split_tokens=self.split_tokens, workspace=self.workspace,
                                out=out, lse=self.lse, k_new=self.k_new, v_new=self.v_new,
                                sinks=self.extra["sinks"], kv_rep=self.cfg.get("kv_rep", 1), plan=self._plan)

    # ---- algorithmic traffic (bytes) --------------------------------------
    def bytes_append(self):
        c = self.cfg
        e = self.q.element_size()
        T = c["B"]
        return 2 * T * (2 * c["Hc"] * c["D"] * e) + 8 * T

    def bytes_decode(self):
        c = self.cfg
        e = self.q.element_size()
        ctx = [L + 1 for L in self.lens]  # the new token attends to itself
        # K rows of every cached head, V rows of every DISTINCT cached head (identical copies count once)
        heads_read = c["Hc"] + c["Hc"] // c.get("kv_rep", 1)
        return (sum(ctx) * heads_read * c["D"] * e + 2 * c["B"] * c["Hq"] * c["D"] * e + 4 * c["B"] * c["Hq"]
                + 8 * sum(math.ceil(x / c["P"]) for x in ctx))


def make_decode_case(name: str, device="cuda", hbm_budget_gb: float | None = None) -> DecodeCase:
    """Seeded decode workload: a fragmented page table built through the public allocator,
    pool, q and the new K/V rows drawn from N(0,1)."""
    from falcon_perception_amd import ops
    from falcon_perception_amd.paged_attention import PagedKVCache

    c = dict(DECODE_WORKLOADS[name])
    dtype = DTYPES[c["dtype"]]
    gen = torch.Generator().manual_seed(c["seed"])
    B, P = c["B"], c["P"]
    lens = [c["prefix"] + int(x) for x in torch.randint(c["lo"], c["hi"] + 1, (B,), generator=gen)]
    need_pages = sum(math.ceil((L + 1) / P) for L in lens) + 1
    n_pages = c["n_pages"]
    if n_pages is None:  # cfg5: pool sized to ~180 GB, or to what this GPU can hold
        e = torch.empty((), dtype=dtype).element_size()
        page_bytes = 2 * c["Hc"] * P * c["D"] * e
        budget = (hbm_budget_gb or 180.0) * 1e9
        n_pages = max(need_pages, int(budget // page_bytes))
    assert need_pages <= n_pages, f"{name}: {need_pages} pages needed, pool has {n_pages}"
    c["n_pages"] = n_pages
    # a pool of several hundred thousand pages gets a sparse page table (columns = blocks of the longest
    # sequence): the reference's dense [B + 1, n_pages] int64 pair would be 1.4 GB at cfg5
    cols = math.ceil((max(lens) + 1) / P) if DECODE_WORKLOADS[name]["n_pages"] is None else None
    cache = PagedKVCache(n_pages, P, B + 1, c["Hc"], c["D"], 1, dtype, device=device, max_blocks_per_seq=cols)
    perm = (torch.randperm(n_pages - 1, generator=gen) + 1).tolist()
    cache.free_pages = perm
    slots = []
    for L in lens:
        b = cache.allocate()
        cache.reserve(b, torch.tensor([b], device=device), L + 1)
        slots.append(b)
    dgen = torch.Generator(device=device).manual_seed(c["seed"])
    flat = cache.kv_cache.view(-1)
    step = 1 << 28
    for s in range(0, flat.numel(), step):  # N(0,1) in place, chunked: no second copy of a 180 GB pool
        flat[s:s + step].normal_(generator=dgen)
    q = torch.randn((B, c["Hq"], 1, c["D"]), generator=dgen, device=device, dtype=torch.float32).to(dtype)
    k_new = torch.randn((B, c["Hc"], 1, c["D"]), generator=dgen, device=device, dtype=torch.float32).to(dtype)
    v_new = torch.randn((B, c["Hc"], 1, c["D"]), generator=dgen, device=device, dtype=torch.float32).to(dtype)
    max_context = min(n_pages * P, math.ceil((max(lens) + 1) / P) * P)
    case = DecodeCase(name, c, cache, lens, torch.tensor(slots, dtype=torch.int64, device=device),
                      torch.tensor(lens, dtype=torch.int32, device=device), q, k_new, v_new, max_context)
    case.split_tokens = ops.decode_split_tokens(B, c["Hc"] // c.get("kv_rep", 1), max_context, P)
    need = ops.decode_workspace_bytes(B, c["Hq"], c["D"], max_context, case.split_tokens)
    case.workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    case.out = torch.empty_like(q)
    case.lse = torch.empty((B, c["Hq"], 1), dtype=torch.float32, device=device)
    case.plan = torch.zeros(ops.decode_plan_bytes(), dtype=torch.uint8, device=device)
    case.make_plan()  # launches that are timed alone (events, single-step graphs) read the plan of this step
    return case


PREFILL_WORKLOADS = {
    # BASELINE.json configs[2]: image prefix already paged, 512-token causal text chunk per sequence
    "cfg3": dict(seed=3, dtype="bf16", n_seq=8, Hq=16, Hc=8, D=128, P=128, prefix_lo=256, prefix_hi=4096, chunk=512),
    # whole sequences in one step (prefix 0): the image span rows are bidirectional
    "cfg3w": dict(seed=3, dtype="bf16", n_seq=8, Hq=16, Hc=8, D=128, P=128, prefix_lo=256, prefix_hi=4096, chunk=512,
                  whole=True),
    # one request alone: a 512-token chunk over a 4096-token prefix (32 workgroups before the cut along the keys)
    "cfg3one": dict(seed=3, dtype="bf16", n_seq=1, Hq=16, Hc=8, D=128, P=128, prefix_lo=4096, prefix_hi=4096, chunk=512),
    # cfg3 in the reference's default dtype (reference server/config.py:38)
    "cfg3f32": dict(seed=3, dtype="f32", n_seq=8, Hq=16, Hc=8, D=128, P=128, prefix_lo=256, prefix_hi=4096, chunk=512),
    # cfg3 on the cache the reference's engine builds: one cached head per query head (paged_inference.py:321-330)
    "cfg3x": dict(seed=3, dtype="bf16", n_seq=8, Hq=16, Hc=16, D=128, P=128, prefix_lo=256, prefix_hi=4096, chunk=512),
    # cfg3 at the head_dim of the OCR and 300M variants
    "cfg3d64": dict(seed=3, dtype="bf16", n_seq=8, Hq=16, Hc=8, D=64, P=128, prefix_lo=256, prefix_hi=4096, chunk=512),
    # whole sequences as the reference's engine prefills them (paged_inference.py:637-672): on its cache of one head per
    # query head, and at head_dim 64
    "cfg3wx": dict(seed=3, dtype="bf16", n_seq=8, Hq=16, Hc=16, D=128, P=128, prefix_lo=256, prefix_hi=4096, chunk=512,
                   whole=True),
    "cfg3wd64": dict(seed=3, dtype="bf16", n_seq=8, Hq=16, Hc=8, D=64, P=128, prefix_lo=256, prefix_hi=4096, chunk=512,
                     whole=True),
}


@dataclass
class PrefillCase:
    """One chunked-prefill step's operands, all on the device."""

    name: str
    cfg: dict
    cache: object
    slots: list
    prefixes: list
    batch_idx: torch.Tensor   # [1, Lq] int64
    input_pos: torch.Tensor   # [1, Lq] int64
    row_limit: torch.Tensor   # [Lq] int32
    q: torch.Tensor
    k_new: torch.Tensor
    v_new: torch.Tensor
    pairs: int                # allowed (q, kv) pairs per head
    # max |q| * max |k| / sqrt(D) over the rows of the case: a bound of |scale * q.k| that holds for this data
    # (the model's normalised q and k have sqrt(D) by construction; N(0, 1) rows are measured)
    score_bound: float = 0.0
    use_bound: bool = True
    input_ids: torch.Tensor | None = None   # [1, Lq] int64 token ids the row limits follow from
    # the step's query tiles by decreasing key range (fp_paged_prefill_tile_order): made once per step, as the row
    # limits are, and taken by every layer's launch; only at head_dim 64, where the order of the workgroups matters
    tile_order: tuple | None = None
    use_order: bool = True

    @property
    def page_size(self):
        return self.cache.page_size

    @property
    def page_table(self):
        return self.cache.page_table

    @property
    def pool_k(self):
        return self.cache.kv_cache[0, 0, 0]

    @property
    def pool_v(self):
        return self.cache.kv_cache[0, 1, 0]

    def append(self):
        self.cache.insert_kv(0, self.k_new, self.v_new, input_pos=self.input_pos, batch_idx=self.batch_idx)

    def attend(self, bounded: bool | None = None):
        from falcon_perception_amd import ops

        bounded = self.use_bound if bounded is None else bounded
        return ops.paged_prefill(self.q, self.pool_k, self.pool_v, self.cache.page_table, self.batch_idx,
                                 self.row_limit, self.page_size,
                                 workspace=self.cache.prefill_workspace(self.q.shape[2], self.q.shape[1], self.q.shape[3],
                                                                        self.pool_k.shape[0], self.q.dtype),
                                 score_bound=self.score_bound if bounded else 0.0,
                                 tile_order=self.tile_order if self.use_order else None)

    def make_tile_order(self):
        """What a model does once per prefill step, next to the mask: rank the step's query tiles."""
        from falcon_perception_amd import ops

        Lq, Hq, D, Hc = self.q.shape[2], self.q.shape[1], self.q.shape[3], self.pool_k.shape[0]
        ws = self.cache.prefill_workspace(Lq, Hq, D, Hc, self.q.dtype)
        rows = ops.prefill_tile_rows(Lq, Hq, Hc, D, self.q.dtype, ws.numel() if ws is not False else 0)
        self.tile_order = ops.prefill_tile_order(self.batch_idx, self.row_limit, rows) if rows else None

    def run(self):
        self.append()
        return self.attend()

    def flops(self):
        return 4 * self.cfg["D"] * self.cfg["Hq"] * self.pairs


def make_prefill_case(name: str, device="cuda") -> PrefillCase:
    from falcon_perception_amd.paged_attention import PagedKVCache

    c = dict(PREFILL_WORKLOADS[name])
    dtype = DTYPES[c["dtype"]]
    gen = torch.Generator().manual_seed(c["seed"])
    P, chunk, n_seq = c["P"], c["chunk"], c["n_seq"]
    prefixes = [int(x) for x in torch.randint(c["prefix_lo"], c["prefix_hi"] + 1, (n_seq,), generator=gen)]
    n_pages = sum(math.ceil((p + chunk) / P) for p in prefixes) + 64
    cache = PagedKVCache(n_pages, P, n_seq + 1, c["Hc"], c["D"], 1, dtype, device=device)
    cache.free_pages = (torch.randperm(n_pages - 1, generator=gen) + 1).tolist()
    slots = []
    for p in prefixes:
        b = cache.allocate()
        cache.reserve(b, torch.tensor([b], device=device), p + chunk)
        slots.append(b)
    dgen = torch.Generator(device=device).manual_seed(c["seed"])
    cache.kv_cache.view(-1).normal_(generator=dgen)
    whole = c.get("whole", False)
    bidx, pos, lim, ids, pairs = [], [], [], [], 0
    for b, p in zip(slots, prefixes):
        if whole:  # all p + chunk rows in this step; rows of the image span [0, p) see the whole span
            n = p + chunk
            row_pos = list(range(n))
            row_lim = [max(t + 1, p) if t < p else t + 1 for t in range(n)]
            row_ids = [SOI_ID] + [IMG_ID] * (p - 1) + [EOI_ID] + [TXT_ID] * (chunk - 1)
        else:      # only the chunk's rows; prefix already cached
            n = chunk
            row_pos = list(range(p, p + chunk))
            row_lim = [t + 1 for t in row_pos]
            row_ids = [TXT_ID] * chunk
        gap = (-n) % 128
        bidx += [b] * n + [0] * gap
        pos += row_pos + [0] * gap
        lim += row_lim + [0] * gap
        ids += row_ids + [PAD_ID] * gap
        pairs += sum(row_lim)
    Lq = len(bidx)
    q = torch.randn((1, c["Hq"], Lq, c["D"]), generator=dgen, device=device, dtype=torch.float32).to(dtype)
    k_new = torch.randn((1, c["Hc"], Lq, c["D"]), generator=dgen, device=device, dtype=torch.float32).to(dtype)
    v_new = torch.randn((1, c["Hc"], Lq, c["D"]), generator=dgen, device=device, dtype=torch.float32).to(dtype)
    k_norm = max(float(cache.kv_cache[0, 0, 0].float().norm(dim=-1).max()), float(k_new.float().norm(dim=-1).max()))
    bound = float(q.float().norm(dim=-1).max()) * k_norm / math.sqrt(c["D"])
    return PrefillCase(name, c, cache, slots, prefixes,
                       torch.tensor([bidx], dtype=torch.int64, device=device),
                       torch.tensor([pos], dtype=torch.int64, device=device),
                       torch.tensor(lim, dtype=torch.int32, device=device), q, k_new, v_new, pairs,
                       score_bound=bound, input_ids=torch.tensor([ids], dtype=torch.int64, device=device))


# --------------------------------------------------------------------------
# timing
# --------------------------------------------------------------------------

def time_steps(fn, steps: int, warmup: int, samples: int = 21) -> float:
    """Wall-clock ms per step of `fn`: a sample is exactly `steps` launches back to back, synchronised on
    both sides; the median of `samples` such regions is returned (after a clock warm-up and `warmup`
    untimed steps)."""
    warm_clocks(fn)
    for _ in range(warmup):
        fn()
    regions = []
    for _ in range(samples):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        regions.append((time.perf_counter() - t0) * 1e3 / steps)
    return statistics.median(regions)


def warm_clocks(fn, seconds: float = 0.2) -> None:
    """Run `fn` back to back for a while: after an idle spell the shader clock needs some tens of
    milliseconds of load to come up, and a handful of warm-up calls would be timed on the ramp
    (a 560 us kernel measured 620 us that way)."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()


def event_ms(fn, steps: int, batch: int = 1) -> float:
    """Device ms per call of `fn`: HIP events on the stream the kernels run on, median of at least 20
    samples.  A sample brackets `batch` back-to-back calls (result divided by `batch`): around a single
    launch the two event markers themselves add 1.5-4 us to what the kernel trace of rocprofv3 reports for
    the kernel, around ten launches a tenth of that."""
    warm_clocks(fn)
    n = max(steps, 20)
    stream = torch.cuda.current_stream()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
    for i in range(n):
        starts[i].record(stream)
        for _ in range(batch):
            fn()
        ends[i].record(stream)
    torch.cuda.synchronize()
    return statistics.median(s.elapsed_time(e) for s, e in zip(starts, ends)) / batch


def graph_ms(fn, steps: int) -> float:
    """ms per step when the step is replayed from a captured HIP graph (how the engine runs decode)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    g.replay()
    torch.cuda.synchronize()
    warm_clocks(g.replay)
    regions = []
    for _ in range(11):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            g.replay()
        torch.cuda.synchronize()
        regions.append((time.perf_counter() - t0) * 1e3 / steps)
    return statistics.median(regions)


def short_kernel_ms(fn, reps: int = 20) -> float:
    """ms per launch of a kernel too short to time through Python (a library call costs the host about 10 us, and
    events around it measure that): `reps` launches back to back in one captured graph, replayed."""
    def many():
        for _ in range(reps):
            fn()

    return graph_ms(many, 20) / reps


def model_depth_graph_ms(case: "DecodeCase", steps: int, layers: int = MODEL_LAYERS) -> float | None:
    """ms for the fused decode step of ALL layers of the model, replayed from one captured HIP graph: every
    layer has its own K/V planes (the same page table, as in the engine) so nothing is served from cache
    between layers.  None when the planes do not fit next to the case's own pool."""
    from falcon_perception_amd import ops

    c = case.cfg
    plane = case.pool_k.numel() * case.pool_k.element_size()
    free, _ = torch.cuda.mem_get_info()
    if 2 * plane * layers > free - (8 << 30):
        return None
    pools = torch.empty((layers, 2) + tuple(case.pool_k.shape), dtype=case.pool_k.dtype, device=case.pool_k.device)
    for layer in range(layers):
        pools[layer, 0].copy_(case.pool_k)
        pools[layer, 1].copy_(case.pool_v)

    def all_layers():
        if case.planned:
            case.make_plan()  # once per step of the model, inside the graph
        for layer in range(layers):
            ops.paged_decode(case.q, pools[layer, 0], pools[layer, 1], case.cache.page_table, case.batch_idx,
                             case.input_pos, case.page_size, case.max_context, split_tokens=case.split_tokens,
                             workspace=case.workspace, out=case.out, lse=case.lse, k_new=case.k_new, v_new=case.v_new,
                             kv_rep=c.get("kv_rep", 1), plan=case._plan)

    ms = graph_ms(all_layers, max(steps // 10, 5))
    del pools
    torch.cuda.empty_cache()  # hand the 56 GiB back: later allocations carved out of it measured 15 % slower copies
    return ms


def append_gather_rates(steps: int = 20, T: int = 32768, H: int = 16, D: int = 128, P: int = 128) -> dict:
    """KV append and page gather at a prefill-sized batch of tokens (the engine's prefill limit,
    reference paged_inference.py:233): bf16, 16 stored heads, one fragmented page table."""
    from falcon_perception_amd import ops
    from falcon_perception_amd.paged_attention import PagedKVCache

    dev, dtype = "cuda", torch.bfloat16
    cache = PagedKVCache(T // P + 16, P, 4, H, D, 1, dtype, device=dev)
    g = torch.Generator().manual_seed(7)
    cache.free_pages = (torch.randperm(cache.n_pages - 1, generator=g) + 1).tolist()
    b = cache.allocate()
    cache.reserve(b, torch.tensor([b], device=dev), T)
    # the model hands K/V over as [1, L, H, D] memory viewed as [1, H, L, D] (reference model.py:118-119)
    k = torch.randn((1, T, H, D), device=dev, dtype=dtype).permute(0, 2, 1, 3)
    v = torch.randn((1, T, H, D), device=dev, dtype=dtype).permute(0, 2, 1, 3)
    bidx = torch.full((1, T), b, dtype=torch.int64, device=dev)
    pos = torch.arange(T, dtype=torch.int64, device=dev)[None]
    pk, pv = cache.kv_cache[0, 0, 0], cache.kv_cache[0, 1, 0]
    k_rows, v_rows = k[0].transpose(0, 1).unsqueeze(2), v[0].transpose(0, 1).unsqueeze(2)
    flat_b, flat_p = bidx.reshape(T), pos.reshape(T, 1)

    def do_append():
        ops.kv_append(pk, pv, k_rows, v_rows, cache.page_table, flat_b, flat_p, P, clamp_negative=False)

    lens = torch.tensor([T], device=dev)
    slots = torch.tensor([b], device=dev)
    out = torch.empty((1, H, T, D), dtype=dtype, device=dev)

    def do_gather():
        ops.kv_gather(pk, cache.page_table, slots, lens, P, T, out=out)

    for _ in range(3):
        do_append()
        do_gather()
    ms_a = event_ms(do_append, steps, batch=5)
    ms_g = event_ms(do_gather, steps, batch=5)
    e = 2
    bytes_a = 2 * T * (2 * H * D * e) + 8 * T
    bytes_g = 2 * T * (H * D * e)
    # the same append over the first t tokens, from a decode step's worth of rows up to the whole batch
    sweep = {}
    for t in (64, 512, 4096, T):
        def do_part(t=t):
            ops.kv_append(pk, pv, k_rows[:t], v_rows[:t], cache.page_table, flat_b[:t], flat_p[:t], P,
                          clamp_negative=False)
        ms_t = event_ms(do_part, steps)
        sweep[str(t)] = {"ms": ms_t, "gbps": (2 * t * (2 * H * D * e) + 8 * t) / (ms_t * 1e-3) / 1e9}

    # The same append and gather with nothing left in the last-level cache from the launch before: six
    # pools, six sets of source rows and six outputs taken in turn (3 GiB / 1.5 GiB touched between two
    # uses of the same addresses, against 256 MB of cache).  The figures above rewrite one pool from one
    # set of rows and gather one pool into one output.
    rings = [(pk, pv, k_rows, v_rows, cache.page_table, out)]
    for i in range(5):
        c2 = PagedKVCache(T // P + 16, P, 4, H, D, 1, dtype, device=dev)
        c2.free_pages = (torch.randperm(c2.n_pages - 1, generator=g) + 1).tolist()
        b2 = c2.allocate()
        assert b2 == b
        c2.reserve(b2, torch.tensor([b2], device=dev), T)
        k2 = torch.randn((T, H, D), device=dev, dtype=dtype)
        v2 = torch.randn((T, H, D), device=dev, dtype=dtype)
        rings.append((c2.kv_cache[0, 0, 0], c2.kv_cache[0, 1, 0], k2.unsqueeze(2), v2.unsqueeze(2), c2.page_table,
                      torch.empty_like(out)))
    turn = [0]

    def do_append_cold():
        rk, rv, sk, sv, table, _ = rings[turn[0] % len(rings)]
        turn[0] += 1
        ops.kv_append(rk, rv, sk, sv, table, flat_b, flat_p, P, clamp_negative=False)

    def do_gather_cold():
        rk, _, _, _, table, o = rings[turn[0] % len(rings)]
        turn[0] += 1
        ops.kv_gather(rk, table, slots, lens, P, T, out=o)

    for _ in range(len(rings)):
        do_append_cold()
    ms_cold = event_ms(do_append_cold, 20, batch=len(rings))
    ms_g_cold = event_ms(do_gather_cold, 20, batch=len(rings))
    del rings

    # QK norm + rotary embedding + insert in one launch (reference model.py:110-119 + the append):
    # the qkv projection output of the same step, 16 query heads / 8 kv heads, expanded to the 16 cached heads
    Hkv = H // 2
    qkv = torch.randn((1, T, (H + 2 * Hkv) * D), device=dev, dtype=dtype)
    xq, xk, xv = qkv.split([H * D, Hkv * D, Hkv * D], dim=-1)
    xq, xk, xv = xq.view(1, T, H, D), xk.view(1, T, Hkv, D), xv.view(1, T, Hkv, D)
    ang = torch.rand((1, T, D // 4), device=dev)
    f1 = torch.polar(torch.ones_like(ang), ang)
    ang2 = torch.rand((1, T, H, D // 4), device=dev)
    f2 = torch.polar(torch.ones_like(ang2), ang2)
    q_out = torch.empty((1, H, T, D), dtype=dtype, device=dev)

    def do_rope():
        ops.qkv_norm_rope_append(xq, xk, xv, f1, f2, pk, pv, cache.page_table, flat_b, pos.reshape(T), P,
                                 clamp_negative=False, q_out=q_out)

    for _ in range(3):
        do_rope()
    ms_r = event_ms(do_rope, steps, batch=5)
    # read q, k, v rows and both angle tables once, write q and the expanded K and V rows, token indices
    bytes_r = (T * (H + 2 * Hkv) * D * e + T * (D // 4) * 8 + T * H * (D // 4) * 8
               + T * H * D * e + 2 * T * H * D * e + 16 * T)
    return {"tokens": T, "heads": H, "head_dim": D,
            "algorithmic_bytes": {"kv_append": bytes_a, "kv_gather": bytes_g, "qkv_norm_rope_append": bytes_r},
            # HBM bytes per launch from the rocprofv3 FETCH_SIZE / WRITE_SIZE summaries under profiles/
            "traffic": {"kv_append": profiled_traffic("kv_append", f"{T}x{H}"),
                        "kv_gather": profiled_traffic("kv_gather", f"{T}x{H}"),
                        "qkv_norm_rope_append": profiled_traffic("qkv_rope_append", f"{T}x{H}")},
            "qkv_norm_rope_append_ms": ms_r, "qkv_norm_rope_append_gbps": bytes_r / (ms_r * 1e-3) / 1e9,
            "qkv_norm_rope_append_frac_of_peak": bytes_r / (ms_r * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "kv_append_ms": ms_a, "kv_append_gbps": bytes_a / (ms_a * 1e-3) / 1e9,
            "kv_append_frac_of_peak": bytes_a / (ms_a * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "kv_append_cold_ms": ms_cold, "kv_append_cold_gbps": bytes_a / (ms_cold * 1e-3) / 1e9,
            "kv_append_cold_frac_of_peak": bytes_a / (ms_cold * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "kv_append_by_tokens": sweep,
            "kv_gather_ms": ms_g, "kv_gather_gbps": bytes_g / (ms_g * 1e-3) / 1e9,
            "kv_gather_frac_of_peak": bytes_g / (ms_g * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "kv_gather_cold_ms": ms_g_cold, "kv_gather_cold_gbps": bytes_g / (ms_g_cold * 1e-3) / 1e9,
            "kv_gather_cold_frac_of_peak": bytes_g / (ms_g_cold * 1e-3) / 1e9 / HBM_PEAK_GBPS}


def prefill_rate(steps: int = 10, name: str = "cfg3", bounded: bool = True, both: bool = True) -> dict:
    """Chunked prefill at BASELINE configs[2]: append the 512-token chunks, attend over the paged prefix.
    `bounded`: declare the score bound (bf16); `both`: time the other variant beside it."""
    case = make_prefill_case(name)
    case.use_bound = bounded
    case.append()
    ms_order = ms_no_order = None
    if case.q.shape[3] == 64 and case.q.dtype != torch.float32:
        case.make_tile_order()
        ms_order = short_kernel_ms(case.make_tile_order)
    for _ in range(3):
        case.attend()
    ms = event_ms(case.attend, steps, batch=4)
    if case.tile_order is not None and both:
        case.use_order = False
        ms_no_order = event_ms(case.attend, steps, batch=4)
        case.use_order = True
    ms_a = event_ms(case.append, steps)
    tf = case.flops() / (ms * 1e-3) / 1e12
    ms_unbounded = None
    if case.q.dtype == torch.bfloat16 and bounded and both:  # the same launch without the score bound: online softmax with a running maximum
        ms_unbounded = event_ms(lambda: case.attend(bounded=False), steps, batch=4)
    what = {"cfg3": "cfg3: 8 sequences, paged prefix U[256,4096], 512-token chunk each, 16 q / 8 kv heads, D 128",
            "cfg3w": "cfg3w: the same 8 sequences prefilled whole (prefix + chunk rows in one step, prefix rows see "
                     "their whole image span), 16 q / 8 kv heads, D 128",
            "cfg3wx": "cfg3w on the reference engine's cache: one cached head per query head (16 q / 16 cached heads)",
            "cfg3wd64": "cfg3w at head_dim 64",
            "cfg3f32": "cfg3 in fp32",
            "cfg3x": "cfg3 on the reference engine's cache: one cached head per query head (16 q / 16 cached heads)",
            "cfg3d64": "cfg3 at head_dim 64 (the reference's OCR and 300M variants)",
            "cfg3one": "one sequence alone: paged prefix 4096, 512-token chunk, 16 q / 8 kv heads, D 128 "
                       "(cut along the keys into 8 shares + merge pass)"}[name]
    # key tiles (64 keys) each 128-row query tile walks: a launch of about one workgroup per CU lasts as long as
    # its longest workgroup, so longest / mean bounds what such a launch can reach of a balanced one's rate
    lim = case.row_limit.view(-1, 128).max(dim=1).values.float()
    tiles = torch.ceil(lim[lim > 0] / 64)
    res = {"workload": what, "query_rows": int(case.q.shape[2]), "paged_prefill_ms": ms, "tflops": tf,
           "chunk_append_ms": ms_a, "flops": case.flops(),
           "key_tiles_per_query_tile": {"longest": int(tiles.max()), "mean": round(float(tiles.mean()), 1),
                                        "query_tiles_per_head": int(tiles.numel())}}
    if ms_order is not None:
        res["tile_order"] = ("workgroups start longest key range first: fp_paged_prefill_tile_order once per step, outside "
                             "the timed launch as the row limits are")
        res["tile_order_kernel_ms"] = ms_order
        res["paged_prefill_ms_no_tile_order"] = ms_no_order
    if case.q.dtype == torch.float32:
        res["frac_of_f32_mfma_peak"] = tf / MFMA_F32_PEAK_TFLOPS
    else:
        res["frac_of_bf16_mfma_peak"] = tf / MFMA_BF16_PEAK_TFLOPS
    if ms_unbounded is not None:
        # the primary figure declares score_bound (a bound of |scale * q.k| measured on the rows of the case; the
        # model's normalised q and k satisfy sqrt(D) by construction); this one leaves it out
        res["score_bound"] = round(case.score_bound, 2)
        res["paged_prefill_ms_no_score_bound"] = ms_unbounded
        res["tflops_no_score_bound"] = case.flops() / (ms_unbounded * 1e-3) / 1e12
    return res


def prefill_drop_in(steps: int = 5, name: str = "cfg3w", layers: int = MODEL_LAYERS) -> dict:
    """A whole prefill step of the model's depth through the callables an unedited engine binds: one
    `create_prefill_blockmask` from the token ids, then `insert_kv` + `compiled_flex_attn_prefill` for every layer
    (reference paged_inference.py:637-733, model.py:150-162).  Wall clock with the host's part in it: Python,
    ctypes, the row-limit kernel, the torch ops that turn packed limits into logical ones."""
    from torch.nn.attention.flex_attention import AuxRequest

    from falcon_perception_amd import attention as A
    from falcon_perception_amd import ops
    from falcon_perception_amd.paged_attention import PagedKVCache

    one = make_prefill_case(name)
    c = one.cfg
    cache = PagedKVCache(one.cache.n_pages, c["P"], c["n_seq"] + 1, c["Hc"], c["D"], layers, DTYPES[c["dtype"]],
                         device=one.q.device, qk_normalised=False)
    cache.page_table.copy_(one.cache.page_table)
    cache.page_table_cpu = [list(r) for r in one.cache.page_table_cpu]
    cache.capacity = list(one.cache.capacity)
    q, k_new, v_new, bidx, pos, ids = one.q, one.k_new, one.v_new, one.batch_idx, one.input_pos, one.input_ids
    flops, bound, limits = one.flops(), one.score_bound, one.row_limit
    del one
    aux = AuxRequest(lse=True)
    state = {}

    def step():
        mask = cache.create_prefill_blockmask(bidx, ids, SOI_ID, EOI_ID)
        for layer in range(layers):
            K, V = cache.insert_kv(layer, k_new, v_new, input_pos=pos, batch_idx=bidx)
            A.compiled_flex_attn_prefill(q, K, V, block_mask=mask, return_aux=aux)
        state["mask"] = mask

    cache.score_bound = lambda head_dim, scale: bound  # what install(qk_norm=True) declares, for these N(0, 1) rows
    step()
    torch.cuda.synchronize()
    real = bidx.view(-1) != 0  # padding rows (slot 0) are never looked at by the kernel
    assert torch.equal(state["mask"].row_limit(pos, 0)[real], limits[real]), "the mask's row limits differ from the hand-written ones"
    ms = time_steps(step, steps, 2, samples=7)
    ms_mask = event_ms(lambda: cache.create_prefill_blockmask(bidx, ids, SOI_ID, EOI_ID), 20)
    ms_limits = event_ms(lambda: ops.hybrid_row_limits(ids, SOI_ID, EOI_ID, bidx), 20, batch=4)
    cache.check_prefill_masks()
    res = {"workload": f"{name}: one prefill step of {layers} layers through create_prefill_blockmask, insert_kv and "
                       "compiled_flex_attn_prefill (Python callables, eager, no host wait in the mask construction)",
           "query_rows": int(q.shape[2]), "ms_per_step": ms, "ms_per_layer": ms / layers,
           "tflops": layers * flops / (ms * 1e-3) / 1e12,
           "frac_of_bf16_mfma_peak": layers * flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
           "create_prefill_blockmask_ms": ms_mask, "hybrid_row_limits_kernel_ms": ms_limits}
    del cache
    torch.cuda.empty_cache()
    return res


def decode_drop_in(case: "DecodeCase", steps: int, model_layers: bool = False) -> dict:
    """The decode layer-step as an unedited engine runs it: `convert_logical_block_mask` once, then `insert_kv` +
    `compiled_flex_attn_decode` (reference paged_inference.py:832-863, model.py:150-162), replayed from a captured
    HIP graph; with the append left to the attention launch (what `install()` switches on) and launched on its own."""
    from torch.nn.attention.flex_attention import AuxRequest, BlockMask

    from falcon_perception_amd import attention as A

    cache, B = case.cache, case.q.shape[0]
    n_blocks = case.max_context // cache.page_size
    full = cache.create_causal_blockmask(B=1, L=n_blocks * cache.page_size)
    blk = (case.input_pos // cache.page_size).long()
    zero = torch.zeros(B, dtype=torch.int64, device=case.q.device)
    logical = BlockMask.from_kv_blocks(
        full.kv_num_blocks[zero, :, blk].view(B, 1, 1), full.kv_indices[zero, :, blk].view(B, 1, 1, -1),
        full.full_kv_num_blocks[zero, :, blk].view(B, 1, 1), full.full_kv_indices[zero, :, blk].view(B, 1, 1, -1),
        BLOCK_SIZE=full.BLOCK_SIZE, mask_mod=lambda b, h, q, kv: q + case.input_pos[b] >= kv,
        seq_lengths=(1, full.seq_lengths[1]))
    aux = AuxRequest(lse=True)
    pos = case.input_pos.view(B, 1)
    saved = (cache.kv_rep, cache.fuse_decode_append)
    cache.kv_rep = case.cfg.get("kv_rep", 1)

    def step(layers=1):
        mask = cache.convert_logical_block_mask(logical, case.batch_idx)
        for _ in range(layers):
            K, V = cache.insert_kv(0, case.k_new, case.v_new, input_pos=pos, batch_idx=case.batch_idx)
            res = A.compiled_flex_attn_decode(case.q, K, V, block_mask=mask, return_aux=aux)
        return res

    res = {}
    for fused in (True, False):
        cache.fuse_decode_append = fused
        res["ms_hip_graph_append_in_attention" if fused else "ms_hip_graph_append_launch"] = graph_ms(step, steps)
    cache.fuse_decode_append = True
    res["ms_eager_append_in_attention"] = time_steps(step, steps, 10, samples=7)
    if model_layers:
        # A step of the whole model: one mask (and so one plan of the decode launches) for all layers, as the engine
        # converts its mask once per step.  The layers here share layer 0's planes; a layer streams more bytes than
        # the last-level cache holds, so no layer is served from what the one before it read.
        ms = graph_ms(lambda: step(MODEL_LAYERS), max(steps // 10, 5))
        res["ms_per_layer_hip_graph_of_all_layers"] = ms / MODEL_LAYERS
    cache.kv_rep, cache.fuse_decode_append = saved
    cache.flush()
    return res


def small_batch_decode(steps: int = 200) -> dict:
    """The decode step (append + split-K pass + merge pass) of a few long sequences, replayed from a HIP
    graph: the regime of one or a few requests, where the split length and the merge pass set the time."""
    out = {}
    for B, L in ((1, 8192), (1, 32768), (4, 8192), (16, 8192)):
        name = f"small_B{B}_L{L}"
        DECODE_WORKLOADS[name] = dict(seed=7, dtype="bf16", B=B, Hq=16, Hc=8, D=128, P=128,
                                      n_pages=B * (L // 128 + 2) + 8, prefix=L - 64, lo=0, hi=63)
        case = make_decode_case(name)
        ms = graph_ms(case.run_fused, steps)
        # one step per replay pays the replay's own launch cost (about 5 us) on a 12 us step; the engine replays a
        # graph of the model's depth, so the same step is also timed as one of 28 layers (own K/V planes each)
        ms_model = model_depth_graph_ms(case, steps)
        out[f"batch {B}, context ~{L}"] = {"split_tokens": case.split_tokens, "ms_per_step_hip_graph": ms,
                                          "gbps": case.bytes_decode() / (ms * 1e-3) / 1e9,
                                          "ms_per_layer_in_a_graph_of_all_layers": ms_model / MODEL_LAYERS if ms_model else None}
        if (B, L) == (1, 8192):  # the same step through the callables an unedited engine binds
            out[f"batch {B}, context ~{L}"]["drop_in"] = decode_drop_in(case, steps)
        del DECODE_WORKLOADS[name], case
        torch.cuda.empty_cache()
    return out


def decode_leg(name: str, steps: int = 50, hbm_budget_gb: float | None = None, cpu: bool = False,
               plan: str = "both") -> dict:
    """One more decode workload next to the headline: the fused step (append inside the split-K pass + merge)
    timed like the headline, the split-K pass alone by events, both priced with the workload's algorithmic
    bytes."""
    if name == "cfg5" and hbm_budget_gb is None:
        free, _ = torch.cuda.mem_get_info()
        hbm_budget_gb = min(180.0, (free - 24e9) / 1e9)
        if hbm_budget_gb < 30:
            return {"skipped": f"only {free / 1e9:.0f} GB of HBM free: no room for a long-context pool"}
    case = make_decode_case(name, hbm_budget_gb=hbm_budget_gb)
    c = case.cfg
    case.planned = plan != "off"
    ms_step = time_steps(case.run_step, steps, 10)
    ms_partial = event_ms(lambda: case.attend("partial"), steps, batch=10)
    ms_unplanned = None if case.planned else ms_step
    if plan == "both":
        case.planned = False
        ms_unplanned = time_steps(case.run_fused, steps, 10, samples=7)
        case.planned = True
    alg_decode, alg_append = case.bytes_decode(), case.bytes_append()
    gbps = (alg_decode + alg_append) / (ms_step * 1e-3) / 1e9
    kernel_gbps = alg_decode / (ms_partial * 1e-3) / 1e9
    res = {
        "workload": f"batch {c['B']}, {c['Hq']} q / {c['Hc']} cached heads"
                    + (f" (V read once per {c['kv_rep']} heads)" if c.get("kv_rep", 1) > 1 else "")
                    + f", head_dim {c['D']}, {c['dtype']}, page_size {c['P']}, {c['n_pages']}-page pool "
                    f"({case.cache.kv_cache.numel() * case.cache.kv_cache.element_size() / 1e9:.1f} GB), contexts "
                    f"{c['prefix']}+U[{c['lo']},{c['hi']}]",
        "ms_per_step": ms_step, "gbps": gbps, "pct_of_hbm_peak": 100.0 * gbps / HBM_PEAK_GBPS,
        "ms_per_step_without_plan": ms_unplanned,
        "decode_tok_s_per_layer": c["B"] / (ms_step * 1e-3), "algorithmic_bytes": alg_decode + alg_append,
        "roofline": {"bound": "hbm", "kernel": "paged_decode_kernel", "achieved": kernel_gbps, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": kernel_gbps / HBM_PEAK_GBPS, "ms": ms_partial,
                     "traffic": profiled_traffic("paged_decode", name), "algorithmic_bytes": alg_decode},
    }
    if cpu:
        res["cpu_baseline"] = cpu_baseline(case, budget_s=5.0, min_reps=20)
        res["gpu_over_cpu"] = gbps / res["cpu_baseline"]["value"]
    del case
    torch.cuda.empty_cache()
    return res


def cfg4_mixed_step(steps: int = 6) -> dict:
    """BASELINE configs[3] as one mixed step: the fused decode step of the running sequences (contexts
    U[512, 8192]) plus the append and chunked-prefill attention of 4 chunks of 1024 tokens (2 fresh sequences
    whose first 512 tokens are an image span, 2 continuing after a 2048-token paged prefix), page size 64,
    16 q / 8 kv heads, D 128, bf16, 8192-page pool.  Between steps the chunk sequences leave and a quarter of
    the decode sequences is erased and replaced through the allocator, so the page tables stay fragmented;
    that host-side churn (and the prefill of the newcomers' contexts) lies outside the timed region."""
    from falcon_perception_amd import ops
    from falcon_perception_amd.paged_attention import PagedKVCache

    dev, dtype = "cuda", torch.bfloat16
    P, Hq, Hc, D, n_pages = 64, 16, 8, 128, 8192
    gen = torch.Generator().manual_seed(4)
    dgen = torch.Generator(device=dev).manual_seed(4)
    cache = PagedKVCache(n_pages, P, 64, Hc, D, 1, dtype, device=dev)
    cache.free_pages = (torch.randperm(n_pages - 1, generator=gen) + 1).tolist()
    cache.kv_cache.view(-1).normal_(generator=dgen)
    pk, pv = cache.kv_cache[0, 0, 0], cache.kv_cache[0, 1, 0]
    rnd = lambda *shape: torch.randn(shape, generator=dgen, device=dev, dtype=torch.float32).to(dtype)

    def admit(length):
        b = cache.allocate()
        cache.reserve(b, torch.tensor([b], device=dev), length)
        return b

    ctx = {}
    for L in torch.randint(512, 8193, (32,), generator=gen).tolist():
        if cache.can_reserve(L + 64):
            ctx[admit(L + 64)] = L  # the pool already holds N(0,1) rows everywhere
    max_context = 8192 + 64
    samples, work = [], []
    q4, k4, v4 = rnd(1, Hq, 4096, D), rnd(1, Hc, 4096, D), rnd(1, Hc, 4096, D)
    for step in range(steps + 2):
        chunks = []
        for kind in ("fresh", "fresh", "cont", "cont"):
            if kind == "fresh":
                chunks.append((admit(1024), 0, [max(t + 1, 512) for t in range(1024)]))
            else:
                chunks.append((admit(2048 + 1024), 2048, [2048 + t + 1 for t in range(1024)]))
        bidx = torch.cat([torch.full((1024,), s, dtype=torch.int64) for s, _, _ in chunks])[None].to(dev)
        pos = torch.cat([torch.arange(st, st + 1024, dtype=torch.int64) for _, st, _ in chunks])[None].to(dev)
        lims = [x for _, _, l in chunks for x in l]
        lim = torch.tensor(lims, dtype=torch.int32, device=dev)
        slots = sorted(ctx)
        B = len(slots)
        bt = torch.tensor(slots, dtype=torch.int64, device=dev)
        pt = torch.tensor([ctx[s] for s in slots], dtype=torch.int32, device=dev)
        k1, v1, q1 = rnd(B, Hc, 1, D), rnd(B, Hc, 1, D), rnd(B, Hq, 1, D)
        split = ops.decode_split_tokens(B, Hc, max_context, P)
        ws = torch.empty(max(ops.decode_workspace_bytes(B, Hq, D, max_context, split), 16), dtype=torch.uint8, device=dev)
        pws = cache.prefill_workspace(4096, Hq, D, Hc, dtype)
        out1 = torch.empty_like(q1)
        lse1 = torch.empty((B, Hq, 1), dtype=torch.float32, device=dev)
        out4 = torch.empty_like(q4)
        lse4 = torch.empty((1, Hq, 4096), dtype=torch.float32, device=dev)

        # a bound of |scale * q.k| that holds for the rows of this step (N(0, 1) everywhere, stale pages included)
        if step == 0:
            k_norm = float(pk.float().norm(dim=-1).max())
        k_norm = max(k_norm, float(k4.float().norm(dim=-1).max()), float(k1.float().norm(dim=-1).max()))
        bound = float(q4.float().norm(dim=-1).max()) * k_norm / math.sqrt(D)

        def mixed():
            ops.paged_decode(q1, pk, pv, cache.page_table, bt, pt, P, max_context, split_tokens=split, workspace=ws,
                             out=out1, lse=lse1, k_new=k1, v_new=v1)
            cache.insert_kv(0, k4, v4, input_pos=pos, batch_idx=bidx)
            ops.paged_prefill(q4, pk, pv, cache.page_table, bidx, lim, P, out=out4, lse=lse4, workspace=pws,
                              score_bound=bound)

        if step == 0:
            warm_clocks(mixed)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        mixed()
        e1.record()
        torch.cuda.synchronize()
        e = 2
        dec_bytes = (sum(ctx[s] + 1 for s in slots) * 2 * Hc * D * e + 2 * B * Hq * D * e + 4 * B * Hq
                     + 8 * sum(math.ceil((ctx[s] + 1) / P) for s in slots) + 2 * B * 2 * Hc * D * e + 8 * B)
        app_bytes = 2 * 4096 * 2 * Hc * D * e + 8 * 4096
        flops = 4 * D * Hq * sum(lims)
        if step >= 2:  # the first two steps are warm-up
            samples.append(e0.elapsed_time(e1))
            work.append((B, dec_bytes, app_bytes, flops))
        for s in slots:
            ctx[s] += 1
        for s, _, _ in chunks:
            cache.erase(s)
        leaving = [slots[i] for i in torch.randperm(B, generator=gen)[: B // 4].tolist()]
        for s in leaving:
            cache.erase(s)
            del ctx[s]
        for L in torch.randint(512, 8193, (len(leaving),), generator=gen).tolist():
            if cache.can_reserve(L + 64):
                ctx[admit(L + 64)] = L
    ms = statistics.median(samples)
    B, dec_bytes, app_bytes, flops = work[samples.index(ms)] if ms in samples else work[-1]
    return {"workload": "cfg4: fused decode step of the running sequences + append and chunked-prefill attention of "
                        "4 x 1024-token chunks, one quarter of the decode sequences replaced between steps",
            "steps_timed": len(samples), "ms_per_mixed_step": ms, "decode_sequences": B,
            "decode_bytes": dec_bytes, "chunk_append_bytes": app_bytes, "prefill_flops": flops,
            "ms_samples": samples}


def cpu_baseline(case: DecodeCase, budget_s: float = 20.0, min_reps: int = 3) -> dict:
    """The reference's op sequence for one decode layer-step, ported to torch-CPU, timed on the
    host cores on a batch subset sized to roughly `budget_s` seconds."""
    from oracle import cpu_path

    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    c = case.cfg
    n = min(c["B"], 4)
    kv = case.cache.kv_cache.cpu().float()  # upcast once, outside the timed region
    pt = case.cache.page_table.cpu()
    p2l = case.cache.physical_to_logical.cpu()

    def one(nb):
        sl = slice(0, nb)
        return cpu_path.decode_step_cpu(kv, 0, pt, p2l, case.batch_idx[sl].cpu(), case.input_pos[sl].cpu(),
                                        case.k_new[sl].cpu().float(), case.v_new[sl].cpu().float(), case.q[sl].cpu().float(),
                                        case.page_size)

    t0 = time.perf_counter()
    one(n)
    probe = time.perf_counter() - t0
    per_seq = probe / n
    nb = int(max(1, min(c["B"], (budget_s / 3) / max(per_seq, 1e-6))))
    times, total = [], 0.0
    while len(times) < min_reps or (len(times) < 20 and total < budget_s):
        t0 = time.perf_counter()
        one(nb)
        times.append(time.perf_counter() - t0)
        total += times[-1]
        if total > 1.5 * budget_s:
            break
    reps, sec = len(times), statistics.median(times)
    ctx = [L + 1 for L in case.lens[:nb]]
    e = case.q.element_size()
    alg = (sum(ctx) * 2 * c["Hc"] * c["D"] * e + 2 * nb * c["Hq"] * c["D"] * e + 4 * nb * c["Hq"]
           + 8 * sum(math.ceil(x / c["P"]) for x in ctx) + 2 * nb * 2 * c["Hc"] * c["D"] * e + 8 * nb)
    return {
        "value": alg / sec / 1e9, "unit": "GB/s", "cores": cores, "cpu": cpu_model(), "kind": "port",
        "sample": f"{nb} of {c['B']} sequences of {case.name}, median of {reps} repetitions, one layer-step each "
                  f"(append + block-id gather + dense masked attention over the whole pool, fp32)",
        "decode_tok_s_per_layer": nb / sec, "ms_per_step_sample": sec * 1e3,
    }


def row_limits_rate(L: int, steps: int = 50) -> dict:
    """The row-limit kernel behind `create_prefill_blockmask` alone, on a packed row of L tokens: sequences of
    4096 tokens, each an image block of 3000 tokens and text, with their cache slots."""
    from falcon_perception_amd import ops

    ids = torch.full((L,), TXT_ID, dtype=torch.int64, device="cuda")
    bidx = torch.ones(L, dtype=torch.int64, device="cuda")
    for s0 in range(0, L, 4096):
        ids[s0] = SOI_ID
        ids[s0 + 1:s0 + 3000] = IMG_ID
        ids[min(s0 + 3000, L - 1)] = EOI_ID
        bidx[s0:s0 + 4096] = 1 + s0 // 4096
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    ms = event_ms(lambda: ops.hybrid_row_limits(ids, SOI_ID, EOI_ID, bidx, None, status), steps, batch=4)
    return {"kernel": "hybrid_row_limits_kernel", "rows": L, "ms": ms, "status": int(status.item())}


def shader_clock_mhz() -> float | None:
    """Current shader clock of GPU 0 as the driver reports it (the starred level of pp_dpm_sclk), or None."""
    import glob

    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
        try:
            with open(path) as f:
                for line in f:
                    if line.rstrip().endswith("*"):
                        return float(line.split(":")[1].strip().split("M")[0])
        except (OSError, ValueError, IndexError):
            continue
    return None


def clock_probe(seconds: float = 2.0) -> dict:
    """Launches of identical prefill workgroups -- n sequences of a 512-row chunk over a 4096-token prefix, 32
    workgroups each, not cut along the keys -- back to back for `seconds` per size, with the shader clock read
    from the driver every 50 ms meanwhile: what a launch of the same workgroups costs as more of the chip is busy."""
    import threading

    from falcon_perception_amd import ops

    out = {}
    for n_seq in (1, 2, 4, 6, 8, 16):
        name = f"probe_{n_seq}"
        PREFILL_WORKLOADS[name] = dict(seed=3, dtype="bf16", n_seq=n_seq, Hq=16, Hc=8, D=128, P=128, prefix_lo=4096,
                                       prefix_hi=4096, chunk=512)
        case = make_prefill_case(name)
        case.append()
        run = lambda: ops.paged_prefill(case.q, case.pool_k, case.pool_v, case.cache.page_table, case.batch_idx,
                                        case.row_limit, case.page_size, workspace=False, score_bound=case.score_bound)
        clocks, stop = [], threading.Event()

        def sample():
            while not stop.is_set():
                mhz = shader_clock_mhz()
                if mhz is not None:
                    clocks.append(mhz)
                time.sleep(0.05)

        warm_clocks(run)
        th = threading.Thread(target=sample)
        th.start()
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(50):
                run()
            torch.cuda.synchronize()
            n += 50
        dt = time.perf_counter() - t0
        stop.set()
        th.join()
        out[f"{32 * n_seq} workgroups"] = {
            "us_per_launch": dt / n * 1e6, "tflops": case.flops() / (dt / n) / 1e12,
            "sclk_mhz_median": statistics.median(clocks) if clocks else None,
            "sclk_mhz_min": min(clocks) if clocks else None, "sclk_samples": len(clocks)}
        del PREFILL_WORKLOADS[name], case
        torch.cuda.empty_cache()
    return out


def overlap_probe(iters: int = 2000) -> dict:
    """`fp_probe_mfma_softmax`: the matrix instructions and the softmax arithmetic of one 64-key tile of the bf16
    prefill kernel (head_dim 128, score bound), stripped of everything else, alone and in turn, with 1 to 3
    wavefronts per SIMD, on a quarter of the CUs (the shader clock stays at its maximum there) and on all of them.
    Reported per slot (one wavefront's tile) and SIMD, in ns and in cycles of the clock read from the driver while
    the launches run."""
    from falcon_perception_amd import _native as N

    lib = N.lib()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = torch.empty(cus * 768, dtype=torch.float32, device="cuda")
    stream = N.stream_ptr(out.device)
    res = {"what": "ns (cycles) per slot and SIMD; a slot = 32 v_mfma_f32_32x32x16_bf16 + softmax of 32 scores per lane",
           "iters": iters, "mfma_cycles_at_peak": 32 * 32}
    for label, wgs in (("quarter_of_the_cus", max(cus // 4, 1)), ("all_cus", cus)):
        leg = {"workgroups": wgs}
        for mode, name in ((0, "matrix_only"), (1, "vector_only"), (2, "both_in_turn")):
            for waves in (1, 2, 3):
                def launch():
                    N.check(lib.fp_probe_mfma_softmax(mode, waves, wgs, iters, out.data_ptr(), out.numel(), stream),
                            "fp_probe_mfma_softmax")

                # launches back to back for about half a second; the clock is read while the second half of them
                # runs, the time is that of the last ten
                launch()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                launch()
                e1.record()
                torch.cuda.synchronize()
                n = max(int(500.0 / max(e0.elapsed_time(e1), 0.05)), 20)
                marks = [torch.cuda.Event(enable_timing=True) for _ in range(11)]
                half = torch.cuda.Event()
                for i in range(n):
                    if i == n // 2:
                        half.record()
                    if i >= n - 10:
                        marks[i - (n - 10)].record()
                    launch()
                marks[10].record()
                half.synchronize()
                clocks = []
                while not marks[10].query():
                    mhz = shader_clock_mhz()
                    if mhz:
                        clocks.append(mhz)
                    time.sleep(0.002)
                torch.cuda.synchronize()
                ms = marks[0].elapsed_time(marks[10]) / 10.0
                ns = ms * 1e6 / (2.0 * iters * waves)
                mhz = statistics.median(clocks) if clocks else None
                leg[f"{name}_{waves}_waves_per_simd"] = {
                    "ns_per_slot": round(ns, 1), "sclk_mhz": mhz,
                    "cycles_per_slot": round(ns * mhz / 1e3) if mhz else None}
        res[label] = leg
    return res


def cpu_model() -> str:
    """Model name of the host processor, as /proc/cpuinfo states it."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def summary_of(result: dict) -> dict:
    """The figures of every leg in a few lines, as the LAST key of the output line: what is kept of a long line is
    its end."""
    def us(x):
        return None if x is None else round(x * 1e3, 1)

    def pct(x):
        return None if x is None else round(100.0 * x, 1)

    out = {"decode_step_us": {}, "decode_step_without_plan_us": {}, "decode_step_pct_of_hbm_peak": {},
           "decode_kernel_pct_of_hbm_peak": {}}
    wl = result["config"]["workload"].split(":")[0]
    out["decode_step_us"][wl] = us(result["ms_per_step"])
    out["decode_step_without_plan_us"][wl] = us(result.get("ms_per_step_without_plan"))
    out["decode_step_pct_of_hbm_peak"][wl] = round(result["pct_of_hbm_peak"], 1)
    out["decode_kernel_pct_of_hbm_peak"][wl] = pct(result["roofline"]["frac"])
    for name, leg in result.get("workloads", {}).items():
        if "ms_per_step" in leg:
            out["decode_step_us"][name] = us(leg["ms_per_step"])
            out["decode_step_without_plan_us"][name] = us(leg.get("ms_per_step_without_plan"))
            out["decode_step_pct_of_hbm_peak"][name] = round(leg["pct_of_hbm_peak"], 1)
            out["decode_kernel_pct_of_hbm_peak"][name] = pct(leg["roofline"]["frac"])
    out["decode_step_variants_us"] = {
        "separate_append_launch": us(result.get("ms_per_step_separate_append")),
        "sink_gate_in_merge": us(result.get("ms_per_step_with_sink_gate")),
        "hip_graph": us(result.get("ms_per_step_hip_graph")),
        "plan_kernel": us(result.get("kernels", {}).get("paged_decode_plan_ms")),
        "all_layers_one_graph_per_layer": us(result["ms_all_layers_hip_graph"] / MODEL_LAYERS)
        if result.get("ms_all_layers_hip_graph") else None}
    if "decode_drop_in" in result:
        out["decode_drop_in_us"] = {k: us(v) for k, v in result["decode_drop_in"].items()}
    if "decode_small_batch" in result:
        out["decode_small_batch_us"] = {}
        for k, v in result["decode_small_batch"].items():
            out["decode_small_batch_us"][k] = us(v["ms_per_step_hip_graph"])
            out["decode_small_batch_us"][k + ", per layer in a graph of all layers"] = us(v.get("ms_per_layer_in_a_graph_of_all_layers"))
            if "drop_in" in v:
                out["decode_small_batch_us"][k + " drop-in"] = {a: us(b) for a, b in v["drop_in"].items()}
    out["tok_s"] = {"per_layer": round(result["decode_tok_s_per_layer"]), "model_measured": result.get("decode_tok_s_model_measured")}
    pf = {}
    for key in [k for k in result if k.startswith(("chunked_prefill", "prefill_whole_sequences"))]:
        leg = result[key]
        name = leg["workload"].split(":")[0]
        frac = leg.get("frac_of_bf16_mfma_peak", leg.get("frac_of_f32_mfma_peak"))
        pf[name] = {"us": us(leg["paged_prefill_ms"]), "tflops": round(leg["tflops"], 1), "pct_of_mfma_peak": pct(frac)}
        if "paged_prefill_ms_no_score_bound" in leg:
            pf[name]["us_no_score_bound"] = us(leg["paged_prefill_ms_no_score_bound"])
        if leg.get("paged_prefill_ms_no_tile_order"):
            pf[name]["us_no_tile_order"] = us(leg["paged_prefill_ms_no_tile_order"])
    if pf:
        out["prefill"] = pf
    if "prefill_drop_in" in result:
        d = result["prefill_drop_in"]
        out["prefill_drop_in"] = {"us_per_layer": us(d["ms_per_layer"]), "pct_of_mfma_peak": pct(d["frac_of_bf16_mfma_peak"]),
                                  "create_prefill_blockmask_us": us(d["create_prefill_blockmask_ms"]),
                                  "hybrid_row_limits_kernel_us": us(d["hybrid_row_limits_kernel_ms"])}
    if "cfg4_mixed_step" in result:
        out["cfg4_mixed_step_us"] = us(result["cfg4_mixed_step"].get("ms_per_mixed_step"))
    ps = result.get("prefill_sized", {})
    if ps:
        out["pieces_pct_of_hbm_peak"] = {k[:-len("_frac_of_peak")]: pct(v) for k, v in ps.items() if k.endswith("_frac_of_peak")}
    cb = {}
    if "cpu_baseline" in result:
        cb[wl] = {k: result["cpu_baseline"][k] for k in ("value", "unit", "cores", "cpu")}
    for name, leg in result.get("workloads", {}).items():
        if "cpu_baseline" in leg:
            cb[name] = {k: leg["cpu_baseline"][k] for k in ("value", "unit", "cores")}
    if cb:
        out["cpu_baseline"] = cb
    return out


def calibration_copies() -> None:
    """Five launches of a plain elementwise copy of known traffic (1 GiB read, 1 GiB written), so that a
    rocprofv3 --pmc run of this process holds the scale of each counter next to the kernels of interest."""
    src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(5):
        torch.mul(src, 2.0, out=dst)
    torch.cuda.synchronize()
    del src, dst


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cfg2", choices=sorted(DECODE_WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--plan", default="both", choices=["both", "on", "off"],
                    help="the decode step plan (fp_paged_decode_plan once per %d layer-steps): 'both' times the headline "
                         "with it and, next to it, without; 'on' / 'off' run every launch of the process one way (for "
                         "profiling)" % MODEL_LAYERS)
    ap.add_argument("--decode-only", action="store_true",
                    help="only the headline workload: no other configs, no append/gather/prefill measurements")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run a plain 1 GiB elementwise copy (x * 2) a few times, so a rocprofv3 --pmc run of this "
                         "command holds a kernel of known traffic next to the kernels of interest")
    ap.add_argument("--hbm-budget-gb", type=float, default=None, help="pool size for cfg5 (default: what fits, at most 180)")
    ap.add_argument("--prefill-only", default=None, choices=sorted(PREFILL_WORKLOADS),
                    help="time only the chunked-prefill attention of this workload and print its JSON (for profiling)")
    ap.add_argument("--no-score-bound", action="store_true",
                    help="with --prefill-only: leave the score bound out (the online softmax with a running maximum)")
    ap.add_argument("--row-limits-only", type=int, default=None, metavar="ROWS",
                    help="time only the row-limit kernel of create_prefill_blockmask on a packed row of ROWS tokens")
    ap.add_argument("--clock-probe", action="store_true",
                    help="launches of identical prefill workgroups at 32 .. 512 workgroups with the shader clock sampled "
                         "from the driver meanwhile, as JSON")
    ap.add_argument("--overlap-probe", action="store_true",
                    help="the matrix and the softmax instructions of one prefill tile, stripped of everything else, alone and "
                         "in turn with 1 .. 3 wavefronts per SIMD (fp_probe_mfma_softmax), as JSON")
    ap.add_argument("--pieces-only", action="store_true",
                    help="time only KV append, page gather and the fused norm + rotary append at 32768 tokens and print "
                         "their JSON (for profiling)")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; each GPU would own its own pool, page table and "
              "sequences with no exchange, so there is nothing to measure at N > 1.", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the hot path has no CPU implementation.", file=sys.stderr)
        return 1

    from falcon_perception_amd import _native

    _native.lib()  # fail loudly if the HIP library is not built
    if args.pmc_calibration:
        calibration_copies()
    if args.prefill_only:
        print(json.dumps(prefill_rate(max(args.steps, 1), args.prefill_only, bounded=not args.no_score_bound, both=False)))
        return 0
    if args.pieces_only:
        print(json.dumps(append_gather_rates(max(args.steps, 1))))
        return 0
    if args.row_limits_only:
        print(json.dumps(row_limits_rate(args.row_limits_only, max(args.steps, 1))))
        return 0
    if args.clock_probe:
        print(json.dumps(clock_probe()))
        return 0
    if args.overlap_probe:
        print(json.dumps(overlap_probe()))
        return 0
    case = make_decode_case(args.workload, hbm_budget_gb=args.hbm_budget_gb)
    c = case.cfg

    case.planned = args.plan != "off"
    ms_step = time_steps(case.run_step, args.steps, args.warmup)
    ms_unplanned = ms_partial_unplanned = None
    if args.plan == "both":
        case.planned = False  # every launch works its cut out from the positions and the page table itself
        ms_unplanned = time_steps(case.run_fused, args.steps, args.warmup, samples=7)
        ms_partial_unplanned = event_ms(lambda: case.attend("partial"), args.steps, batch=10)
        case.planned = True
    ms_plan = short_kernel_ms(case.make_plan) if case.planned else None
    ms_separate = time_steps(case.run, args.steps, args.warmup, samples=5)
    ms_gated = time_steps(case.run_fused_gated, args.steps, args.warmup, samples=5)
    ms_graph = graph_ms(case.run_fused, args.steps)
    ms_decode = event_ms(case.attend, args.steps)
    ms_partial = event_ms(lambda: case.attend("partial"), args.steps, batch=10)  # the dominant kernel alone
    ms_merge = short_kernel_ms(lambda: case.attend("merge"))
    ms_append = short_kernel_ms(case.append)
    case.attend()

    alg_decode = case.bytes_decode()
    alg_append = case.bytes_append()
    alg_step = alg_decode + alg_append
    value = alg_step / (ms_step * 1e-3) / 1e9
    achieved = alg_decode / (ms_partial * 1e-3) / 1e9

    result = {
        "metric": "paged decode attn + KV append HBM GB/s (% of peak); decode tok/s",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": c["dtype"], "data": "synthetic",
        "config": {"workload": f"{case.name}: decode layer-step, batch {c['B']}, {c['Hq']} q / {c['Hc']} kv heads, "
                               f"head_dim {c['D']}, page_size {c['P']}, {c['n_pages']}-page pool, contexts "
                               f"{c['prefix']}+U[{c['lo']},{c['hi']}], seed {c['seed']}",
                   "tokens_in_cache": sum(case.lens), "split_tokens": case.split_tokens,
                   "step_plan": (f"fp_paged_decode_plan launched once per {MODEL_LAYERS} layer-steps inside the timed region "
                                 "(ms_per_step_without_plan: no plan at all)") if case.planned else "none"},
        "timing": "ms_per_step = median of 21 regions of exactly `steps` back-to-back steps, synchronised on both "
                  "sides; kernel times = median of >= 20 HIP-event samples on the launch stream",
        "pct_of_hbm_peak": 100.0 * value / HBM_PEAK_GBPS,
        "decode_tok_s_per_layer": c["B"] / (ms_step * 1e-3),
        "decode_tok_s_model": c["B"] / (ms_step * 1e-3) / MODEL_LAYERS,
        # measured, not divided: the fused step of all 28 layers (own K/V planes each) in one HIP graph
        "ms_all_layers_hip_graph": None,
        "decode_tok_s_model_measured": None,
        "step": "fp_paged_decode_append (append fused into the split-K pass) + merge pass"
                + (f"; fp_paged_decode_plan once per {MODEL_LAYERS} layer-steps, inside the timed region (a model plans once "
                   "per step for all its layers)" if case.planned else "; no step plan"),
        "ms_per_step_without_plan": ms_unplanned if case.planned else ms_step,
        "value_without_plan": alg_step / (ms_unplanned * 1e-3) / 1e9 if ms_unplanned else None,
        "ms_per_step_separate_append": ms_separate,
        "ms_per_step_with_sink_gate": ms_gated,  # same step, sigmoid(lse - sink) gate + [B,1,H*D] layout in the merge
        "value_separate_append": alg_step / (ms_separate * 1e-3) / 1e9,
        "ms_per_step_hip_graph": ms_graph,
        "value_hip_graph": alg_step / (ms_graph * 1e-3) / 1e9,
        "kernels": {"paged_decode_ms": ms_decode, "paged_decode_partial_ms": ms_partial,
                    "paged_decode_merge_ms": ms_merge, "paged_decode_plan_ms": ms_plan,
                    "paged_decode_partial_without_plan_ms": ms_partial_unplanned,
                    "paged_decode_gbps": alg_decode / (ms_decode * 1e-3) / 1e9,
                    "kv_append_ms": ms_append, "kv_append_gbps": alg_append / (ms_append * 1e-3) / 1e9},
        "roofline": {"bound": "hbm", "kernel": "paged_decode_kernel", "achieved": achieved,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": profiled_traffic("paged_decode", case.name), "algorithmic_bytes": alg_decode},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(case)
        result["gpu_over_cpu"] = value / result["cpu_baseline"]["value"]
    if not args.decode_only:
        result["decode_drop_in"] = decode_drop_in(case, args.steps, model_layers=True)
        ms_model = model_depth_graph_ms(case, args.steps)  # takes and returns 56 GiB
        if ms_model is not None:
            result["ms_all_layers_hip_graph"] = ms_model
            result["decode_tok_s_model_measured"] = c["B"] / (ms_model * 1e-3)
        del case
        torch.cuda.empty_cache()
        # every other BASELINE config, the expanded-head cache of the reference's engine, head_dim 64
        legs = {}
        for name in ("cfg1", "cfg2x", "cfg2xs", "cfg2d64", "cfg2f32", "cfg4d", "cfg5"):
            if name != args.workload:
                legs[name] = decode_leg(name, hbm_budget_gb=args.hbm_budget_gb if name == "cfg5" else None,
                                        cpu=(name == "cfg1" and not args.no_cpu_baseline), plan=args.plan)
        result["workloads"] = legs
        result["cfg4_mixed_step"] = cfg4_mixed_step()
        result["prefill_sized"] = append_gather_rates()
        result["chunked_prefill"] = prefill_rate()
        result["chunked_prefill_expanded_heads"] = prefill_rate(name="cfg3x")
        result["chunked_prefill_head_dim_64"] = prefill_rate(name="cfg3d64")
        result["chunked_prefill_fp32"] = prefill_rate(name="cfg3f32")
        result["chunked_prefill_one_sequence"] = prefill_rate(name="cfg3one")
        result["prefill_whole_sequences"] = prefill_rate(name="cfg3w")
        result["prefill_whole_sequences_expanded_heads"] = prefill_rate(name="cfg3wx")
        result["prefill_whole_sequences_head_dim_64"] = prefill_rate(name="cfg3wd64")
        result["decode_small_batch"] = small_batch_decode()
        result["prefill_drop_in"] = prefill_drop_in()
    result["summary"] = summary_of(result)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
