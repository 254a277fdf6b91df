"""Helpers for attention tests on long contexts: requests laid out in a paged cache on the device, and float64
attention computed there with library products only (one head and a few hundred queries at a time, so that 32k keys
fit).  Nothing here touches the framework's kernels."""
import math

import torch

DEV = "cuda:0"


def reference_attention(q, k, v, q_pos, scale, window=0, chunk=256):
    """float64 attention of q [n, heads, d] (at positions q_pos [n]) over keys and values [L, kv_heads, d] of one
    request: keys 0..position, or the last `window` of them.  Returns float64 [n, heads, d] on q's device."""
    n, heads, d = q.shape
    L, kv_heads = k.shape[0], k.shape[1]
    qd, kd, vd = q.double(), k.double(), v.double()
    out = torch.empty_like(qd)
    kpos = torch.arange(L, device=q.device)
    q_pos = q_pos.to(q.device).long()
    for h in range(heads):
        kh, vh = kd[:, h // (heads // kv_heads)], vd[:, h // (heads // kv_heads)]
        for a in range(0, n, chunk):
            s = (qd[a:a + chunk, h] @ kh.T) * scale
            pos = q_pos[a:a + chunk, None]
            ok = kpos[None, :] <= pos
            if window > 0:
                ok &= kpos[None, :] >= pos + 1 - window
            out[a:a + chunk, h] = torch.softmax(s.masked_fill(~ok, -math.inf), -1) @ vh
    return out


def paged_on_device(seq_lens, q_lens, heads, kv_heads, d, page_size, seed=0, table=None, pages=None):
    """bfloat16 q/k/v for requests of the given context and new-token counts, in a paged cache on the device.
    Pages are handed out in a scrambled order, or as `table` (int [S, width], from a cache manager) says, in a pool
    of `pages` pages.  Returns q, k_cache, v_cache, table, positions, seq_of_token and the dense (k, v) per request."""
    S = len(seq_lens)
    blocks = [-(-L // page_size) for L in seq_lens]
    if table is None:
        total = sum(blocks) + 3
        order = torch.randperm(total, generator=torch.Generator().manual_seed(seed))
        table = torch.full((S, max(blocks) + 1), -1, dtype=torch.int32)
        at = 0
        for s, nb in enumerate(blocks):
            table[s, :nb] = order[at:at + nb].int()
            at += nb
    else:
        table = torch.as_tensor(table).int().reshape(S, -1)
        total = pages
    g = torch.Generator(device=DEV).manual_seed(seed)
    k_cache = torch.zeros(total, kv_heads, page_size, d, dtype=torch.bfloat16, device=DEV)
    v_cache = torch.zeros(total, kv_heads, d, page_size, dtype=torch.bfloat16, device=DEV)
    dense, qs, positions, seq_of_token = [], [], [], []
    for s, (L, n, nb) in enumerate(zip(seq_lens, q_lens, blocks)):
        k = torch.randn(L, kv_heads, d, device=DEV, generator=g).bfloat16()
        v = torch.randn(L, kv_heads, d, device=DEV, generator=g).bfloat16()
        qs.append(torch.randn(n, heads, d, device=DEV, generator=g).bfloat16())
        dense.append((k, v))
        positions += list(range(L - n, L))
        seq_of_token += [s] * n
    p = dict(q=torch.cat(qs), k_cache=k_cache, v_cache=v_cache, table=table.to(DEV), dense=dense, qs=qs,
             positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
             seq_of_token=torch.tensor(seq_of_token, dtype=torch.int32, device=DEV), page_size=page_size)
    for s in range(S):
        write_request(p, s)
    return p


def write_request(p, s):
    """(Re)writes request s's dense keys and values into its pages."""
    k, v = p["dense"][s]
    page_size = p["page_size"]
    L, kv_heads, d = k.shape
    nb = -(-L // page_size)
    own = p["table"][s, :nb].long()
    kp = torch.zeros(nb * page_size, kv_heads, d, dtype=k.dtype, device=DEV)
    vp = torch.zeros_like(kp)
    kp[:L], vp[:L] = k, v
    p["k_cache"][own] = kp.view(nb, page_size, kv_heads, d).permute(0, 2, 1, 3)
    p["v_cache"][own] = vp.view(nb, page_size, kv_heads, d).permute(0, 2, 3, 1)


def reference_for(p, seq_lens, q_lens, scale, window=0):
    """float64 attention of every request of `paged_on_device`, rows in the step's order."""
    outs = []
    for (k, v), q, L, n in zip(p["dense"], p["qs"], seq_lens, q_lens):
        outs.append(reference_attention(q, k, v, torch.arange(L - n, L), scale, window))
    return torch.cat(outs)


def attention_from_cache(q, k_cache, v_cache, table, q_start, seq_lens, scale, window=0):
    """float64 attention of a step's rows, with keys and values read back from the pages through the block table
    (q [T, heads, d]; q_start [S + 1] and seq_lens [S] on the host): what the cache holds is taken as given, so
    this checks the attention kernels of a running engine and not what wrote the cache."""
    page_size = k_cache.shape[2]
    outs = []
    for s, L in enumerate(int(x) for x in seq_lens):
        a, b = int(q_start[s]), int(q_start[s + 1])
        if a == b:
            continue
        nb = -(-L // page_size)
        first = 0
        if window > 0:  # pages that every query of the step has passed may have been given back (table entry -1)
            first = max(0, (L - (b - a) + 1 - window)) // page_size
        own = table[s, first:nb].long()
        k = k_cache[own].permute(0, 2, 1, 3).reshape((nb - first) * page_size, k_cache.shape[1], -1)
        v = v_cache[own].permute(0, 3, 1, 2).reshape((nb - first) * page_size, k_cache.shape[1], -1)
        pos = torch.arange(L - (b - a), L) - first * page_size
        outs.append(reference_attention(q[a:b], k[:L - first * page_size], v[:L - first * page_size], pos, scale, window))
    return torch.cat(outs)


def rel_err(got, want):
    want = want.double()
    return float((got.double().to(want.device) - want).abs().max()) / max(float(want.abs().max()), 1e-30)
