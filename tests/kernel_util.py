"""Test-side helpers for kernel tests: page packing written independently of the
kernels (from the documented layout), and float64 reference attention."""

from __future__ import annotations

import torch

from tokamak_amd.engine.batch import StepSpan, build_batch
from tokamak_amd.kernels.attention import ATTENTION_WORK


def pack_pages(k_cache, v_cache, k_seq, v_seq, table, ps):
    """Write a request's keys/values ([T, nkv, hd]) into its pages.
    K page: [nkv][hd/8][ps][8]; V page: [nkv][hd/16][ps/4][16][4]."""
    T, nkv, hd = k_seq.shape
    for t in range(T):
        page, off = table[t // ps], t % ps
        kp = k_cache[page].view(nkv, hd // 8, ps, 8)
        vp = v_cache[page].view(nkv, hd // 16, ps // 4, 16, 4)
        kp[:, :, off, :] = k_seq[t].view(nkv, hd // 8, 8).to(k_cache.dtype)
        vp[:, :, off // 4, :, off % 4] = v_seq[t].view(nkv, hd // 16, 16).to(v_cache.dtype)


def pack_pages_whole(k_cache, v_cache, k_seq, v_seq, table, ps):
    """The same layout for a long request without a loop over tokens: the sequence is
    padded to whole pages and permuted page-wise (pinned against ``pack_pages``)."""
    T, nkv, hd = k_seq.shape
    pages = -(-T // ps)
    pad = pages * ps - T
    if pad:
        k_seq = torch.cat([k_seq, torch.zeros(pad, nkv, hd, dtype=k_seq.dtype)])
        v_seq = torch.cat([v_seq, torch.zeros(pad, nkv, hd, dtype=v_seq.dtype)])
    index = torch.tensor(table[:pages])
    kp = k_seq.view(pages, ps, nkv, hd // 8, 8).permute(0, 2, 3, 1, 4)                  # [P][nkv][hd/8][ps][8]
    vp = v_seq.view(pages, ps // 4, 4, nkv, hd // 16, 16).permute(0, 3, 4, 1, 5, 2)      # [P][nkv][hd/16][ps/4][16][4]
    k_cache[index] = kp.reshape(pages, -1).to(k_cache.dtype)
    v_cache[index] = vp.reshape(pages, -1).to(v_cache.dtype)


def unpack_pages(k_cache, v_cache, table, T, nkv, hd, ps):
    k = torch.empty(T, nkv, hd, dtype=k_cache.dtype)
    v = torch.empty(T, nkv, hd, dtype=v_cache.dtype)
    for t in range(T):
        page, off = table[t // ps], t % ps
        k[t] = k_cache[page].view(nkv, hd // 8, ps, 8)[:, :, off, :].reshape(nkv, hd).cpu()
        v[t] = v_cache[page].view(nkv, hd // 16, ps // 4, 16, 4)[:, :, off // 4, :, off % 4].reshape(nkv, hd).cpu()
    return k, v


def reference_attention(q, k, v, positions, scale, window=None):
    """float64, explicit softmax.  q [Tq, nh, hd] at absolute ``positions``;
    k, v [Tk, nkv, hd] (position = index).  Query head a uses kv head a // G."""
    q, k, v = q.double(), k.double(), v.double()
    Tq, nh, hd = q.shape
    group = nh // k.shape[1]
    out = torch.zeros(Tq, nh, hd, dtype=torch.float64)
    for i, p in enumerate(positions):
        lo = 0 if window is None else max(0, p - window + 1)
        for a in range(nh):
            kv = a // group
            s = (k[lo:p + 1, kv] @ q[i, a]) * scale
            w = torch.softmax(s, dim=0)
            out[i, a] = w @ v[lo:p + 1, kv]
    return out


def reference_attention_blocked(q, k, v, positions, scale, block=256):
    """``reference_attention`` for long contexts: float64, explicit softmax, all heads of a
    block of queries at once (no loop over single queries; no window)."""
    q, k, v = q.double(), k.double(), v.double()
    Tq, nh, hd = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    positions = torch.as_tensor(list(positions))
    out = torch.empty(Tq, nh, hd, dtype=torch.float64)
    for a in range(0, Tq, block):
        pos = positions[a:a + block]
        last = int(pos.max()) + 1
        hidden = torch.arange(last)[None, :] > pos[:, None]                     # [B, last]
        for kv in range(nkv):
            heads = slice(kv * group, (kv + 1) * group)
            s = torch.einsum("bgd,td->bgt", q[a:a + block, heads], k[:last, kv]) * scale
            s = s.masked_fill(hidden[:, None, :], float("-inf"))
            w = torch.softmax(s, dim=-1)
            out[a:a + block, heads] = torch.einsum("bgt,td->bgd", w, v[:last, kv])
    return out


def make_batch(spans, device="cuda"):
    """spans: list of (tokens_count, ctx_len, table) -> StepBatch with one cache group and
    the attention kernels' work lists."""
    ss = [StepSpan(request=i, tokens=[0] * n, ctx_len=ctx, state_slot=i, tables=[table])
          for i, (n, ctx, table) in enumerate(spans)]
    return build_batch(ss, 1, device, [ATTENTION_WORK])
