"""GPU: the sequence of cache and attention calls the reference engine makes, replayed against
the oracle.  Follows paged_inference.py: engine init (:321-352), graph capture with temporary
one-page slots (:865-952), packed prefill (:608-733), decode steps through captured HIP graphs
with padded batch buckets (:954-1031, :783-863), page growth and preemption (:1209-1238).  As in
the reference, the capture runs in the constructor, outside inference mode (:434-435), and everything
`generate` does (admission, prefill, decode, growth, erase) runs under `torch.inference_mode()`
(:1331; the server's loop likewise, server/engine_worker.py:126)."""

import numpy as np
import pytest
import torch
from torch.nn.attention.flex_attention import AuxRequest, BlockMask

from falcon_perception_amd import attention as A
from falcon_perception_amd.paged_attention import PagedKVCache
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, f64, randn
from tests.test_oracle_masks import EOI, IMG, PAD, SOI, TXT

pytestmark = pytest.mark.gpu

P, N_PAGES, MAX_BS, MAX_SEQ = 16, 96, 8, 256
H, D, LAYERS = 4, 128, 2
DTYPE = torch.bfloat16
ATOL, RTOL = 2e-2, 1e-2


class MiniEngine:
    """The parts of PagedInferenceEngine that touch the cache, with random K/V/Q instead of a model."""

    def __init__(self, fuse_decode_append=False):
        self.cache = PagedKVCache(N_PAGES, P, MAX_BS, H, D, LAYERS, DTYPE, device=DEV,
                                  fuse_decode_append=fuse_decode_append)
        self.block_mask = self.cache.create_causal_blockmask(B=MAX_BS, L=MAX_SEQ)
        self.input_pos = torch.zeros(MAX_BS, dtype=torch.int32, device=DEV)
        self.gen = torch.Generator().manual_seed(0)
        # oracle mirror
        self.alloc = O.PagedAllocator(N_PAGES, P, MAX_BS)
        self.ref_pool = np.zeros(tuple(self.cache.kv_cache.shape), dtype=np.float64)
        self.graphs = {}

    # -- paged_inference.py:783-826
    def decoding_mask(self, batch_idx, input_pos):
        bm = self.block_mask
        B = batch_idx.shape[0]
        blk = input_pos // bm.BLOCK_SIZE[0]
        return BlockMask.from_kv_blocks(
            bm.kv_num_blocks[batch_idx, :, blk].view(B, 1, 1), bm.kv_indices[batch_idx, :, blk].view(B, 1, 1, -1),
            bm.full_kv_num_blocks[batch_idx, :, blk].view(B, 1, 1),
            bm.full_kv_indices[batch_idx, :, blk].view(B, 1, 1, -1),
            BLOCK_SIZE=bm.BLOCK_SIZE, mask_mod=lambda b, h, q, kv: q + input_pos[b] >= kv,
            seq_lengths=(1, bm.seq_lengths[1]))

    # -- paged_inference.py:832-863, one "model forward" = LAYERS x (insert_kv, attention)
    def decode_forward(self, batch_idx, k, v, q, out, lse):
        B = batch_idx.shape[0]
        pos = self.input_pos[batch_idx]
        mask = self.cache.convert_logical_block_mask(self.decoding_mask(batch_idx, pos), batch_idx)
        for layer in range(LAYERS):
            K, V = self.cache.insert_kv(layer, k[layer, :B], v[layer, :B], input_pos=pos.view(B, 1), batch_idx=batch_idx)
            o, aux = A.compiled_flex_attn_decode(q[layer, :B], K, V, block_mask=mask, return_aux=AuxRequest(lse=True),
                                                 kernel_options={})
            assert self.cache.last_decode_step.k_new is None  # the rows are in the pool, by either route
            out[layer, :B] = o
            lse[layer, :B] = aux.lse

    # -- paged_inference.py:865-952
    def capture(self):
        self.g_bidx = torch.arange(MAX_BS, dtype=torch.int64, device=DEV)
        self.g_k = torch.zeros((LAYERS, MAX_BS, H, 1, D), dtype=DTYPE, device=DEV)
        self.g_v = torch.zeros_like(self.g_k)
        self.g_q = torch.zeros_like(self.g_k)
        self.g_out = torch.zeros_like(self.g_k)
        self.g_lse = torch.zeros((LAYERS, MAX_BS, H, 1), dtype=torch.float32, device=DEV)
        temp = []
        for _ in range(MAX_BS):
            if not self.cache.can_reserve(P):
                break
            slot = self.cache.allocate()
            self.cache.reserve(batch_idx_int=slot, batch_idx=torch.tensor([slot], device=DEV), seq_len=P)
            assert self.alloc.allocate() == slot and self.alloc.reserve(slot, P)
            temp.append(slot)
        assert temp == list(range(1, MAX_BS))  # slot 0 is never handed out
        pool = None
        for bs in (8, 4, 2, 1):
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            self.decode_forward(self.g_bidx[:bs], self.g_k, self.g_v, self.g_q, self.g_out, self.g_lse)  # warm-up
            with torch.cuda.graph(g, pool=pool):
                self.decode_forward(self.g_bidx[:bs], self.g_k, self.g_v, self.g_q, self.g_out, self.g_lse)
            pool = pool or g.pool()
            self.graphs[bs] = g
            torch.cuda.synchronize()
        for slot in temp:
            self.input_pos[slot] = 0
            self.cache.erase(slot)
            self.alloc.erase(slot)
        # the capture runs wrote rows at position 0 of the temporary slots: the pool is scratch until
        # real sequences overwrite it, so the mirror starts from the device state
        self.ref_pool = self.cache.kv_cache.double().cpu().numpy()

    def admit(self, length):
        slot = self.cache.allocate()
        assert slot == self.alloc.allocate()
        self.cache.reserve(batch_idx_int=slot, batch_idx=torch.tensor([slot], device=DEV), seq_len=length)
        self.alloc.reserve(slot, length)
        return slot

    def grow(self, slot, length):
        if self.cache.capacity[slot] >= length:
            return True
        if not self.cache.can_reserve(length, batch_idx_int=slot):
            return False
        self.cache.reserve(batch_idx_int=slot, batch_idx=torch.tensor([slot], device=DEV), seq_len=length)
        self.alloc.reserve(slot, length)
        return True

    def release(self, slot):
        self.cache.erase(slot)
        self.alloc.erase(slot)

    # -- paged_inference.py:608-733: pack, pad each sequence to 128 with (slot 0, pos 0, PAD)
    def prefill(self, seqs):
        ids, bidx, pos = [], [], []
        for slot, tokens in seqs:
            L = len(tokens)
            gap = (-L) % 128
            ids += list(tokens) + [PAD] * gap
            bidx += [slot] * L + [0] * gap
            pos += list(range(L)) + [0] * gap
            self.input_pos[slot] = L - 1
        ids, bidx, pos = np.array(ids), np.array(bidx), np.array(pos)
        Lp = len(ids)
        t = lambda a: torch.from_numpy(a)[None].to(DEV)
        mask = self.cache.create_prefill_blockmask(t(bidx), t(ids), SOI, EOI)
        for layer in range(LAYERS):
            k, v, q = (randn(self.gen, (1, H, Lp, D), DTYPE) for _ in range(3))
            K, V = self.cache.insert_kv(layer, k.to(DEV), v.to(DEV), input_pos=t(pos), batch_idx=t(bidx))
            assert K.shape == (1, H, Lp, D)  # prefill hands the fresh rows back
            out, aux = A.compiled_flex_attn_prefill(q.to(DEV), K, V, block_mask=mask, return_aux=AuxRequest(lse=True),
                                                    kernel_options={"FORCE_USE_FLEX_ATTENTION": True})
            O.append_prefill(self.ref_pool, layer, f64(k), f64(v), self.alloc.page_table, bidx[None], pos[None], P)
            eo, el = O.prefill_attention_packed(f64(q), f64(k), f64(v), bidx[None], ids[None], SOI, EOI)
            real = np.flatnonzero(bidx != 0)
            np.testing.assert_allclose(f64(out)[:, :, real], eo[:, :, real], atol=ATOL, rtol=RTOL)
            np.testing.assert_allclose(f64(aux.lse)[:, :, real], el[:, :, real], atol=2e-3, rtol=RTOL)

    # -- paged_inference.py:954-1031: pick the bucket, pad with slot 0, replay the graph
    def decode(self, slots, lengths):
        B = len(slots)
        bucket = next(b for b in (1, 2, 4, 8) if b >= B)
        padded = torch.zeros(MAX_BS, dtype=torch.int64)
        padded[:B] = torch.tensor(slots)
        self.g_bidx.copy_(padded.to(DEV))
        self.input_pos.scatter_(0, torch.tensor(slots, device=DEV), torch.tensor(lengths, dtype=torch.int32, device=DEV))
        k, v, q = (randn(self.gen, (LAYERS, MAX_BS, H, 1, D), DTYPE) for _ in range(3))
        self.g_k.copy_(k.to(DEV))
        self.g_v.copy_(v.to(DEV))
        self.g_q.copy_(q.to(DEV))
        self.graphs[bucket].replay()
        torch.cuda.synchronize()
        for layer in range(LAYERS):
            O.append_decode(self.ref_pool, layer, f64(k[layer, :B]), f64(v[layer, :B]), self.alloc.page_table,
                            np.array(slots), np.array(lengths)[:, None], P)
            eo, el = O.decode_attention(f64(q[layer, :B]), self.ref_pool[layer, 0, 0], self.ref_pool[layer, 1, 0],
                                        self.alloc.page_table, slots, np.array(lengths), P)
            np.testing.assert_allclose(f64(self.g_out[layer, :B]), eo, atol=ATOL, rtol=RTOL)
            np.testing.assert_allclose(f64(self.g_lse[layer, :B]), el, atol=2e-3, rtol=RTOL)
        assert torch.isfinite(self.g_out.float()).all()  # padded rows read page 0 and stay finite

    def check_pool(self):
        got = self.cache.kv_cache.double().cpu().numpy()
        # page 0 takes padding rows (prefill gaps, graph padding): unspecified contents
        assert np.array_equal(got[..., P:, :], self.ref_pool[..., P:, :])
        assert self.cache.page_table.cpu().numpy().tolist() == self.alloc.page_table.tolist()
        assert self.cache.physical_to_logical.cpu().numpy().tolist() == self.alloc.physical_to_logical.tolist()
        assert self.cache.free_pages == self.alloc.free_pages and self.cache.free_batch_idx == self.alloc.free_batch_idx


def tokens(n_text_before, n_img, n_text_after):
    img = [SOI] + [IMG + 1] * 4 + [IMG] * n_img + [EOI] if n_img else []
    return [TXT] * n_text_before + img + [TXT] * n_text_after


@pytest.mark.parametrize("fuse_decode_append", [False, True], ids=["append-launch", "append-in-attention"])
def test_engine_call_sequence(fuse_decode_append):
    """`fuse_decode_append` is what `install()` switches on for an engine that is not edited: the decode
    `insert_kv` launches nothing and the attention call that follows appends and attends in one kernel.  The
    pool is compared with the oracle's after the attention calls either way."""
    eng = MiniEngine(fuse_decode_append)
    eng.capture()
    with torch.inference_mode():
        generate(eng)


def test_a_decode_append_left_to_the_attention_call_is_launched_by_whatever_comes_first():
    """With `fuse_decode_append` the rows of a decode `insert_kv` wait for the attention call.  Reading
    `kv_cache`, another insert, `erase` or `flush` must find them in the pool."""
    cache = PagedKVCache(8, P, 4, H, D, 2, DTYPE, device=DEV, fuse_decode_append=True)
    slot = cache.allocate()
    cache.reserve(slot, torch.tensor([slot], device=DEV), 3 * P)
    gen = torch.Generator().manual_seed(5)
    bidx = torch.tensor([slot], device=DEV)
    page = cache.page_table_cpu[slot][0]

    def row(layer, pos):
        return cache.kv_cache[layer, 0, 0, :, page * P + pos].clone()

    k, v = (randn(gen, (1, H, 1, D), DTYPE).to(DEV) for _ in range(2))
    cache.insert_kv(0, k, v, input_pos=torch.tensor([[2]], dtype=torch.int32, device=DEV), batch_idx=bidx)
    assert cache.last_decode_step.k_new is k  # nothing launched yet
    assert torch.equal(row(0, 2), k[0, :, 0])  # the property launches the append
    assert cache.last_decode_step.k_new is None
    k2, v2 = (randn(gen, (1, H, 1, D), DTYPE).to(DEV) for _ in range(2))
    cache.insert_kv(0, k2, v2, input_pos=torch.tensor([[3]], dtype=torch.int32, device=DEV), batch_idx=bidx)
    cache.insert_kv(1, k, v, input_pos=torch.tensor([[3]], dtype=torch.int32, device=DEV), batch_idx=bidx)  # next layer first
    assert torch.equal(cache._kv[0, 0, 0, :, page * P + 3], k2[0, :, 0])
    cache.flush()
    assert torch.equal(cache._kv[1, 1, 0, :, page * P + 3], v[0, :, 0])
    cache.insert_kv(0, k2, v2, input_pos=torch.tensor([[4]], dtype=torch.int32, device=DEV), batch_idx=bidx)
    cache.erase(slot)  # the rows land before the slot's pages go back
    assert torch.equal(cache._kv[0, 0, 0, :, page * P + 4], k2[0, :, 0])


def test_kv_rep_from_install_is_checked_against_the_first_prefill(monkeypatch):
    """A cache that took kv_rep from the class default (install(kv_rep=2)) and is then fed V heads that are not
    copies -- a second engine in the process, a model without head repeat -- refuses at its first prefill."""
    monkeypatch.setattr(PagedKVCache, "default_kv_rep", 2)
    gen = torch.Generator().manual_seed(6)
    t = lambda a: torch.tensor([a], device=DEV)
    for copies in (True, False):
        cache = PagedKVCache(8, P, 4, H, D, 1, DTYPE, device=DEV)
        assert cache.kv_rep == 2
        slot = cache.allocate()
        cache.reserve(slot, torch.tensor([slot], device=DEV), 10)
        k = randn(gen, (1, H, 10, D), DTYPE).to(DEV)
        v = randn(gen, (1, H // 2, 10, D), DTYPE).to(DEV).repeat_interleave(2, dim=1) if copies else randn(gen, (1, H, 10, D), DTYPE).to(DEV)
        if copies:
            cache.insert_kv(0, k, v, input_pos=t(list(range(10))), batch_idx=t([slot] * 10))
            assert cache.v_copies_are_identical()
        else:
            with pytest.raises(RuntimeError, match="not 2 identical copies"):
                cache.insert_kv(0, k, v, input_pos=t(list(range(10))), batch_idx=t([slot] * 10))
    explicit = PagedKVCache(8, P, 4, H, D, 1, DTYPE, device=DEV, kv_rep=1)
    assert explicit.kv_rep == 1 and not explicit._kv_rep_unverified


def generate(eng):
    assert torch.is_inference_mode_enabled()
    assert eng.cache.num_free_pages == N_PAGES - 1 and len(eng.cache.free_batch_idx) == MAX_BS - 1

    # step 1: prefill three sequences (image + text, text only, image at position 0)
    prompts = [tokens(3, 40, 10), tokens(20, 0, 0), tokens(0, 25, 60)]
    running = {}
    batch = []
    for tk in prompts:
        slot = eng.admit(len(tk))
        running[slot] = len(tk)
        batch.append((slot, tk))
    eng.prefill(batch)
    eng.check_pool()

    # steps 2..: decode, growing across page boundaries; one more sequence joins, one finishes, one is preempted
    rng = np.random.default_rng(1)
    for step in range(40):
        if step == 5:
            tk = tokens(1, 8, 3)
            slot = eng.admit(len(tk))
            eng.prefill([(slot, tk)])
            running[slot] = len(tk)
        if step == 12:  # the shortest sequence finishes: its pages go back to the free list
            done = min(running, key=running.get)
            eng.release(done)
            del running[done]
        if step == 20:  # preemption (paged_inference.py:1231-1237): newest sequence is erased and re-prefilled later
            newest = max(running)
            eng.release(newest)
            lost = running.pop(newest)
            tk = tokens(0, 0, lost)
            slot = eng.admit(len(tk))
            eng.prefill([(slot, tk)])
            running[slot] = len(tk)
        slots = sorted(running)
        lengths = []
        for s in slots:
            assert eng.grow(s, running[s] + 1)
            lengths.append(running[s])  # the new token goes to position = current length
            running[s] += 1
        eng.decode(slots, lengths)
        if step % 10 == 9:
            eng.check_pool()
    eng.check_pool()
    # pool exhaustion raises exactly like the reference (paged_attention.py:138-143)
    s = sorted(running)[0]
    with pytest.raises(RuntimeError, match="Cannot reserve"):
        eng.cache.reserve(s, torch.tensor([s], device=DEV), N_PAGES * P + 1)
