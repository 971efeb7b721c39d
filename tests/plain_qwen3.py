"""Plain, slow Qwen3 dense: whole sequences, no cache, one function per part.

Written from the reference's formulas; each function cites the lines it
follows (paths relative to the reference checkout).  It shares no code with
``tokamak_amd``: it reads ``config.json`` and ``model.safetensors`` itself and
computes everything on the CPU with torch tensor arithmetic only (no library
attention, no library norm).  All arithmetic runs in the dtype of ``weights``
(float32 by default, float64 on request).
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


# ----------------------------------------------------------------------------
# reading a model folder
# ----------------------------------------------------------------------------
def read_folder(folder: str | Path, dtype: torch.dtype = torch.float32):
    """Return (config dict, {tensor name: tensor in ``dtype``})."""
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    weights = {}
    for file in sorted(folder.glob("*.safetensors")):
        with safe_open(file, framework="pt", device="cpu") as f:
            for name in f.keys():
                weights[name] = f.get_tensor(name).to(dtype)
    return cfg, weights


def sizes(cfg: dict) -> dict:
    """Sizes and constants with the reference's defaults (src/tokamak/config.py:98-125)."""
    nh = int(cfg["num_attention_heads"])
    hd = cfg.get("head_dim")
    if hd is None:
        hd = cfg["hidden_size"] // nh  # src/tokamak/config.py:99-101
    theta = cfg.get("rope_theta")
    if theta is None:
        theta = cfg["rope_parameters"]["rope_theta"]  # src/tokamak/config.py:138-147
    return dict(
        L=int(cfg["num_hidden_layers"]),
        H=int(cfg["hidden_size"]),
        nh=nh,
        nkv=int(cfg.get("num_key_value_heads", nh)),  # src/tokamak/config.py:116
        hd=int(hd),
        I=int(cfg["intermediate_size"]),
        V=int(cfg["vocab_size"]),
        eps=float(cfg["rms_norm_eps"]),
        theta=float(theta),
        tied=bool(cfg.get("tie_word_embeddings", False)),  # src/tokamak/config.py:122
    )


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """src/tokamak/model/layers.py:28-33: x * rsqrt(mean(x^2) + eps), then times weight."""
    variance = (x * x).mean(dim=-1, keepdim=True)
    return weight * (x * torch.rsqrt(variance + eps))


def rope_tables(positions: torch.Tensor, head_dim: int, theta: float):
    """src/tokamak/model/layers.py:47,56-58: inv_freq and angles in float32.

    inv_freq[j] = 1 / theta^(2j/hd); angle = float(pos) * inv_freq; the table is
    the angle list written twice (first half, second half).
    """
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    freqs = positions.to(torch.float32)[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """src/tokamak/model/layers.py:61-63: (x1, x2) -> (-x2, x1), halves not pairs."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """src/tokamak/model/layers.py:81-89: x*cos + rotate_half(x)*sin.

    ``x`` is [T, heads, hd]; tables are [T, hd] and broadcast over heads.
    """
    cos = cos.to(x.dtype)[:, None, :]
    sin = sin.to(x.dtype)[:, None, :]
    return x * cos + rotate_half(x) * sin


def causal_gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                         query_block: int | None = None) -> torch.Tensor:
    """Scores, mask, softmax, weighted values.

    q [T, nh, hd]; k, v [T, nkv, hd].  Query head a uses kv head a // G
    (src/tokamak/kernels/paged_attention.py:74-78; enable_gqa in
    src/tokamak/model/step_context.py:90-92), scale = hd^-0.5
    (src/tokamak/kernels/paged_attention.py:277), a query at position t sees
    positions c <= t (src/tokamak/model/step_context.py:93-96), explicit softmax
    as in tests/unit/test_paged_attention_kernel.py:42-50.

    ``query_block``: for sequences whose [T, T] score matrix would not fit in memory, the
    same arithmetic for ``query_block`` queries at a time against the keys up to the
    block's last query (the keys behind it are masked anyway).
    """
    T, nh, hd = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    out = torch.empty_like(q)
    block = T if query_block is None else query_block
    for first in range(0, T, block):
        last = min(T, first + block)
        visible = torch.arange(last)[None, :] <= torch.arange(first, last)[:, None]
        for a in range(nh):
            kv = a // group
            scores = (q[first:last, a, :] @ k[:last, kv, :].T) * scale
            scores = scores.masked_fill(~visible, float("-inf"))
            scores = scores - scores.max(dim=-1, keepdim=True).values
            probs = scores.exp()
            probs = probs / probs.sum(dim=-1, keepdim=True)
            out[first:last, a, :] = probs @ v[:last, kv, :]
    return out


def attention_block(h: torch.Tensor, w: dict, prefix: str, s: dict, positions: torch.Tensor,
                    query_block: int | None = None) -> torch.Tensor:
    """src/tokamak/model/transformer.py:65-86: project, per-head q/k norm, rope, attend, o_proj."""
    T = h.shape[0]
    q = (h @ w[prefix + "q_proj.weight"].T).view(T, s["nh"], s["hd"])
    k = (h @ w[prefix + "k_proj.weight"].T).view(T, s["nkv"], s["hd"])
    v = (h @ w[prefix + "v_proj.weight"].T).view(T, s["nkv"], s["hd"])
    # per-head norm over hd, before rotation; v is not normed (transformer.py:71-73)
    q = rmsnorm(q, w[prefix + "q_norm.weight"], s["eps"])
    k = rmsnorm(k, w[prefix + "k_norm.weight"], s["eps"])
    cos, sin = rope_tables(positions, s["hd"], s["theta"])
    q = apply_rope(q, cos, sin)
    k = apply_rope(k, cos, sin)
    o = causal_gqa_attention(q, k, v, s["hd"] ** -0.5, query_block)
    return o.reshape(T, s["nh"] * s["hd"]) @ w[prefix + "o_proj.weight"].T


def silu(x: torch.Tensor) -> torch.Tensor:
    """z * sigmoid(z) (src/tokamak/model/layers.py:103 uses F.silu)."""
    return x / (1.0 + torch.exp(-x))


def swiglu(h: torch.Tensor, w: dict, prefix: str) -> torch.Tensor:
    """src/tokamak/model/layers.py:101-104: down(silu(gate(x)) * up(x))."""
    gate = h @ w[prefix + "gate_proj.weight"].T
    up = h @ w[prefix + "up_proj.weight"].T
    return (silu(gate) * up) @ w[prefix + "down_proj.weight"].T


def decoder_layer(x: torch.Tensor, w: dict, i: int, s: dict, positions: torch.Tensor,
                  query_block: int | None = None) -> torch.Tensor:
    """src/tokamak/model/transformer.py:107-108: pre-norm residual block."""
    p = f"model.layers.{i}."
    x = x + attention_block(rmsnorm(x, w[p + "input_layernorm.weight"], s["eps"]), w, p + "self_attn.", s, positions,
                            query_block)
    x = x + swiglu(rmsnorm(x, w[p + "post_attention_layernorm.weight"], s["eps"]), w, p + "mlp.")
    return x


def hidden_states(token_ids, cfg: dict, w: dict, start_position: int = 0,
                  query_block: int | None = None) -> torch.Tensor:
    """src/tokamak/model/transformer.py:138-144: embed, L layers, final norm."""
    s = sizes(cfg)
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    positions = torch.arange(len(ids)) + start_position
    x = w["model.embed_tokens.weight"][ids]  # plain row gather (transformer.py:140)
    for i in range(s["L"]):
        x = decoder_layer(x, w, i, s, positions, query_block)
    return rmsnorm(x, w["model.norm.weight"], s["eps"])


def logits(token_ids, cfg: dict, w: dict, start_position: int = 0, query_block: int | None = None) -> torch.Tensor:
    """Logits [T, V] at every position (src/tokamak/model/transformer.py:173-176).

    A tied model projects with the embedding matrix itself (transformer.py:155-156).
    """
    s = sizes(cfg)
    head = w["model.embed_tokens.weight"] if s["tied"] else w["lm_head.weight"]
    return (hidden_states(token_ids, cfg, w, start_position, query_block) @ head.T).to(torch.float32)


def greedy(token_ids, num_new: int, cfg: dict, w: dict) -> list[int]:
    """Greedy continuation, recomputing the whole sequence each token
    (argmax, first maximum wins: src/tokamak/sampling/sampler.py:58-59)."""
    ids = list(token_ids)
    out = []
    for _ in range(num_new):
        nxt = int(torch.argmax(logits(ids, cfg, w)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out


# ----------------------------------------------------------------------------
# sampling (src/tokamak/sampling/sampler.py:17-84)
# ----------------------------------------------------------------------------
def sampling_probs(row: torch.Tensor, temperature: float, top_k: int, top_p: float) -> torch.Tensor:
    """Distribution after temperature -> top-k -> top-p (sampler.py:34-39)."""
    x = row.to(torch.float64) / temperature
    V = x.numel()
    if 0 < top_k < V:  # sampler.py:35-36,64-67: ties at the k-th value survive
        kth = torch.sort(x, descending=True).values[top_k - 1]
        x = torch.where(x < kth, torch.full_like(x, -math.inf), x)
    if top_p < 1.0:  # sampler.py:70-84
        order = torch.argsort(x, descending=True, stable=True)
        sx = x[order]
        p = torch.exp(sx - sx.max())
        p = p / p.sum()
        before = torch.cumsum(p, 0) - p
        sx = torch.where(before >= top_p, torch.full_like(sx, -math.inf), sx)
        x = torch.full_like(x, -math.inf)
        x[order] = sx
    p = torch.exp(x - x.max())
    return p / p.sum()
