"""torch-CPU port of the reference's paged decode step (TEST / BASELINE INFRASTRUCTURE).

Runs the same sequence of tensor operations the reference executes for one layer
of one decode step, on the host cores, in float32:

  1. KV append by advanced-index assignment          (paged_attention.py:212-230)
  2. logical -> physical block ids (zeros + gather)    (paged_attention.py:279-284)
  3. dense attention over the WHOLE pool with the physical-space mask
     `valid(page) & (q_pos >= logical_kv)`             (paged_attention.py:303-333,
     paged_inference.py:797-801), softmax and LSE as torch's eager math_attention
     does for an uncompiled flex_attention call
     (torch/_higher_order_ops/flex_attention.py:202-268).

This is what `bench.py` times as `cpu_baseline` (kind "port"); tests check it
against the numpy oracle.  The product package never imports it.
"""

from __future__ import annotations

import math

import torch


def decode_step_cpu(kv_cache, layer, page_table, physical_to_logical, batch_idx, input_pos,
                    k_new, v_new, q, page_size, logical_kv_indices=None):
    """One layer of one decode step on CPU tensors.

    kv_cache [L, 2, 1, Hc, N, D]; batch_idx [B] int64; input_pos [B] int; k_new, v_new
    [B, Hc, 1, D]; q [B, Hq, 1, D].  Returns (out [B, Hq, 1, D] float32, lse [B, Hq, 1]).
    """
    B, Hq, _, D = q.shape
    Hc = kv_cache.shape[3]
    N = kv_cache.shape[4]
    n_pages = N // page_size
    pos = input_pos.view(B, 1).to(torch.int64)

    # 1. append
    phys = torch.gather(page_table[batch_idx], 1, pos // page_size).to(torch.int32).clamp(min=0)
    addr = (phys * page_size + (pos % page_size)).view(-1)
    kv_cache[layer, 0, :, :, addr, :] = k_new.permute(1, 0, 2, 3).contiguous().view(1, Hc, B, D)
    kv_cache[layer, 1, :, :, addr, :] = v_new.permute(1, 0, 2, 3).contiguous().view(1, Hc, B, D)
    K = kv_cache[layer, 0]  # [1, Hc, N, D]
    V = kv_cache[layer, 1]

    # 2. block-id conversion of the step's logical block list
    if logical_kv_indices is not None:
        conv = torch.zeros((B, 1, 1, n_pages), dtype=torch.int32)
        C = logical_kv_indices.shape[-1]
        conv[..., :C] = torch.gather(page_table[batch_idx], 1, logical_kv_indices.view(B, -1).long()) \
            .view(B, 1, 1, C).to(torch.int32)

    # 3. dense masked attention over every physical slot
    slot = torch.arange(N)
    block = physical_to_logical[batch_idx][:, slot // page_size]  # [B, N]
    logical = block * page_size + slot % page_size
    mask = (block >= 0) & (pos >= logical.clamp(min=0))  # [B, N]
    G = Hq // Hc
    Kf = K[0].float()  # no copy when the pool is already float32
    Vf = V[0].float()
    qg = q[:, :, 0].float().view(B, Hc, G, D)  # query head h reads cache head h // G
    scores = torch.einsum("bhgd,hnd->bhgn", qg, Kf) / math.sqrt(D)
    scores = scores.masked_fill(~mask[:, None, None, :], float("-inf"))
    lse = torch.logsumexp(scores, dim=-1)
    p = torch.exp(scores - lse[..., None]).nan_to_num(0.0)
    out = torch.einsum("bhgn,hnd->bhgd", p, Vf)
    return out.reshape(B, Hq, 1, D), lse.reshape(B, Hq, 1)
