"""Pins of the plain implementation beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine, and
invariants, each chosen so that a plausible mistake fails it.

The reference's own top test compares its model with the `transformers`
implementation on a downloaded checkpoint (tests/integration/test_hf_parity.py:25-96).
Neither a checkpoint nor another project's model code is used here, so parity
with that implementation is unpinned; what stands in its place are the library
compositions below (F.linear, F.rms_norm, F.scaled_dot_product_attention with its
default scale, F.silu), which fix the scale, the place and value of eps, and which
tensors are normed."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain
from tiny import TINIES, make_folder


# -- RMSNorm (reference tests/unit/test_layers.py:11-27) ----------------------
def test_rmsnorm_formula_and_unit_rms():
    torch.manual_seed(0)
    w = torch.randn(64)
    x = torch.randn(2, 5, 64)
    expected = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w
    torch.testing.assert_close(plain.rmsnorm(x, w, 1e-6), expected, rtol=1e-5, atol=1e-6)
    out = plain.rmsnorm(torch.randn(10, 128) * 3.0, torch.ones(128), 1e-8)
    torch.testing.assert_close(out.pow(2).mean(-1).sqrt(), torch.ones(10), rtol=1e-3, atol=1e-3)
    # scale invariance (eps -> 0): a norm that forgot the rsqrt, or used the mean, fails
    torch.testing.assert_close(plain.rmsnorm(7.0 * x, w, 1e-12), plain.rmsnorm(x, w, 1e-12), rtol=1e-5, atol=1e-6)


def test_rmsnorm_eps_sits_inside_the_root():
    """Inputs so small that eps (1e-5) is ten times mean(x^2) (1e-6): with eps added
    outside the root the result is 2.8 times larger, with eps left out 3.3 times.
    Closed form, and the library routine that the form reduces to."""
    torch.manual_seed(10)
    eps = 1e-5
    x = torch.randn(7, 96, dtype=torch.float64) * 1e-3
    w = 1.0 + 0.1 * torch.randn(96, dtype=torch.float64)
    ms = (x * x).sum(-1, keepdim=True) / 96
    assert 0.5e-6 < float(ms.mean()) < 2e-6
    expected = x / torch.sqrt(ms + eps) * w
    got = plain.rmsnorm(x, w, eps)
    torch.testing.assert_close(got, expected, rtol=1e-12, atol=0)
    torch.testing.assert_close(got, F.rms_norm(x, (96,), w, eps), rtol=1e-12, atol=0)
    outside = x / (torch.sqrt(ms) + eps) * w
    assert float((outside.abs() / got.abs()).min()) > 2.0          # what the test would catch


# -- RoPE (reference tests/unit/test_layers.py:30-68) -------------------------
def test_rope_position_zero_is_identity_and_norm_is_kept():
    cos, sin = plain.rope_tables(torch.tensor([0]), 32, 10000.0)
    q = torch.randn(1, 4, 32)
    torch.testing.assert_close(plain.apply_rope(q, cos, sin), q)
    cos, sin = plain.rope_tables(torch.arange(10), 64, 1e6)
    q = torch.randn(10, 4, 64)
    torch.testing.assert_close(plain.apply_rope(q, cos, sin).norm(dim=-1), q.norm(dim=-1), rtol=1e-4, atol=1e-4)


def test_rope_dot_depends_on_distance_only():
    torch.manual_seed(3)
    q, k = torch.randn(1, 1, 32), torch.randn(1, 1, 32)

    def dot(m, n):
        cq, sq = plain.rope_tables(torch.tensor([m]), 32, 10000.0)
        ck, sk = plain.rope_tables(torch.tensor([n]), 32, 10000.0)
        return float((plain.apply_rope(q, cq, sq) * plain.apply_rope(k, ck, sk)).sum())

    assert abs(dot(5, 3) - dot(9, 7)) < 1e-4
    assert abs(dot(10, 0) - dot(15, 5)) < 1e-4
    assert abs(dot(5, 3) - dot(3, 5)) > 1e-3      # the sign of the distance matters


def test_rope_pairs_halves_not_neighbours_and_turns_the_right_way():
    hd, theta, pos = 8, 10000.0, 3
    cos, sin = plain.rope_tables(torch.tensor([pos]), hd, theta)
    x = torch.zeros(1, 1, hd)
    x[0, 0, 1] = 1.0                                # unit vector on dim 1
    out = plain.apply_rope(x, cos, sin)[0, 0]
    angle = pos * theta ** (-2.0 / hd)              # frequency index 1
    expected = torch.zeros(hd)
    expected[1] = math.cos(angle)                   # stays on dim 1 ...
    expected[1 + hd // 2] = math.sin(angle)         # ... and leaks into dim 1 + hd/2 with a plus sign
    torch.testing.assert_close(out, expected, rtol=1e-5, atol=1e-6)


# -- attention core ------------------------------------------------------------
def test_attention_equals_library_sdpa_with_gqa():
    torch.manual_seed(1)
    T, nh, nkv, hd = 11, 6, 3, 16
    q, k, v = torch.randn(T, nh, hd), torch.randn(T, nkv, hd), torch.randn(T, nkv, hd)
    ours = plain.causal_gqa_attention(q, k, v, hd ** -0.5)
    rep = nh // nkv
    lib = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1).repeat_interleave(rep, 0)[None],
        v.transpose(0, 1).repeat_interleave(rep, 0)[None], is_causal=True)[0].transpose(0, 1)
    torch.testing.assert_close(ours, lib, rtol=1e-5, atol=1e-5)


def test_attention_special_cases():
    torch.manual_seed(2)
    nh, nkv, hd = 4, 2, 8
    q, k, v = torch.randn(1, nh, hd), torch.randn(1, nkv, hd), torch.randn(1, nkv, hd)
    out = plain.causal_gqa_attention(q, k, v, hd ** -0.5)
    # one token: softmax over one key is 1, the output is v of head a // G (not a % nkv)
    torch.testing.assert_close(out[0, 0], v[0, 0])
    torch.testing.assert_close(out[0, 1], v[0, 0])
    torch.testing.assert_close(out[0, 2], v[0, 1])
    torch.testing.assert_close(out[0, 3], v[0, 1])
    # all keys equal: output is the mean of the visible values
    T = 6
    q, v = torch.randn(T, nh, hd), torch.randn(T, nkv, hd)
    k = torch.randn(1, nkv, hd).expand(T, nkv, hd)
    out = plain.causal_gqa_attention(q, k, v, hd ** -0.5)
    for t in range(T):
        torch.testing.assert_close(out[t, 3], v[: t + 1, 1].mean(0), rtol=1e-5, atol=1e-6)


def test_attention_scale_is_applied_to_scores():
    torch.manual_seed(4)
    T, hd = 5, 8
    q, k, v = torch.randn(T, 1, hd), torch.randn(T, 1, hd), torch.randn(T, 1, hd)
    a = plain.causal_gqa_attention(q, k, v, 0.5)
    b = plain.causal_gqa_attention(q * 0.5, k, v, 1.0)
    torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)


# -- SwiGLU (reference tests/unit/test_layers.py:71-79) -----------------------
def test_swiglu_zero_gate_and_library_silu():
    torch.manual_seed(5)
    w = {"gate_proj.weight": torch.randn(32, 16), "up_proj.weight": torch.randn(32, 16),
         "down_proj.weight": torch.randn(16, 32)}
    x = torch.randn(3, 16)
    lib = (F.silu(x @ w["gate_proj.weight"].T) * (x @ w["up_proj.weight"].T)) @ w["down_proj.weight"].T
    torch.testing.assert_close(plain.swiglu(x, w, ""), lib, rtol=1e-5, atol=1e-5)
    w["gate_proj.weight"] = torch.zeros(32, 16)
    torch.testing.assert_close(plain.swiglu(x, w, ""), torch.zeros(3, 16))


# -- whole model -----------------------------------------------------------------
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("plain")
    return {k: plain.read_folder(make_folder(root, k)) for k in ("A", "B")}


def test_layers_switched_off_leave_head_of_norm_of_embedding(folders):
    cfg, w = folders["B"]
    w = dict(w)
    for i in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.o_proj.weight"] = torch.zeros_like(w[f"model.layers.{i}.self_attn.o_proj.weight"])
        w[f"model.layers.{i}.mlp.down_proj.weight"] = torch.zeros_like(w[f"model.layers.{i}.mlp.down_proj.weight"])
    ids = [3, 1, 4, 1, 5]
    emb = w["model.embed_tokens.weight"][torch.tensor(ids)]
    expected = plain.rmsnorm(emb, w["model.norm.weight"], cfg["rms_norm_eps"]) @ w["lm_head.weight"].T
    torch.testing.assert_close(plain.logits(ids, cfg, w), expected, rtol=1e-5, atol=1e-6)


def test_causality(folders):
    cfg, w = folders["A"]
    ids = [5, 9, 2, 7, 11, 3, 8]
    base = plain.logits(ids, cfg, w)
    changed = plain.logits(ids[:-1] + [200], cfg, w)
    torch.testing.assert_close(base[:-1], changed[:-1], rtol=0, atol=0)
    assert (base[-1] - changed[-1]).abs().max() > 1e-4


def test_shift_of_all_positions_changes_nothing(folders):
    # only distances count: a rotation with the wrong sign on k, or applied to v, fails this
    for key in ("A", "B"):
        cfg, w = folders[key]
        ids = list(range(10, 22))
        a = plain.logits(ids, cfg, w, start_position=0)
        b = plain.logits(ids, cfg, w, start_position=37)
        torch.testing.assert_close(a, b, rtol=1e-4, atol=2e-5)


def test_tied_head_uses_the_embedding(folders):
    cfg, w = folders["A"]
    assert cfg["tie_word_embeddings"] and "lm_head.weight" not in w
    h = plain.hidden_states([1, 2, 3], cfg, w)
    torch.testing.assert_close(plain.logits([1, 2, 3], cfg, w), h @ w["model.embed_tokens.weight"].T)


def test_qk_norm_comes_before_rotation(folders):
    cfg, w = folders["B"]
    s = plain.sizes(cfg)
    torch.manual_seed(6)
    h = torch.randn(4, s["H"])
    p = "model.layers.0.self_attn."
    w1 = dict(w)
    w1[p + "q_norm.weight"] = torch.ones(s["hd"])
    q = (h @ w1[p + "q_proj.weight"].T).view(4, s["nh"], s["hd"])
    qn = plain.rmsnorm(q, w1[p + "q_norm.weight"], 0.0)
    cos, sin = plain.rope_tables(torch.arange(4), s["hd"], s["theta"])
    rotated = plain.apply_rope(qn, cos, sin)
    torch.testing.assert_close(rotated.norm(dim=-1), torch.full((4, s["nh"]), math.sqrt(s["hd"])), rtol=1e-4, atol=1e-4)


def _library_attention_block(h, w, p, cfg, positions):
    """The attention sub-layer put together from library routines only: F.linear,
    F.rms_norm over the head axis with the model's eps, and
    F.scaled_dot_product_attention with its DEFAULT scale, which is
    1/sqrt(q.size(-1)), the size of a head as q is laid out, whatever hidden/heads is.
    Only the rotation comes from the plain implementation (pinned on its own above)."""
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    T = h.shape[0]
    q = F.rms_norm(F.linear(h, w[p + "q_proj.weight"]).view(T, nh, hd), (hd,), w[p + "q_norm.weight"], eps)
    k = F.rms_norm(F.linear(h, w[p + "k_proj.weight"]).view(T, nkv, hd), (hd,), w[p + "k_norm.weight"], eps)
    v = F.linear(h, w[p + "v_proj.weight"]).view(T, nkv, hd)
    cos, sin = plain.rope_tables(positions, hd, float(cfg["rope_theta"]))
    q, k = plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin)
    rep = nh // nkv
    o = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1).repeat_interleave(rep, 0)[None],
        v.transpose(0, 1).repeat_interleave(rep, 0)[None], is_causal=True)[0].transpose(0, 1)
    return F.linear(o.reshape(T, nh * hd), w[p + "o_proj.weight"])


def test_attention_block_equals_library_composition_with_default_scale(folders):
    """Configuration B has head_dim 32 while hidden/heads is 16: a softmax scale taken
    from hidden/heads differs by sqrt(2) in every score and fails this.  The scores
    are made large enough (q and k norm weights times 3, so |score| reaches ~10)
    that the softmax is far from uniform and the scale shows in the output."""
    cfg, w = folders["B"]
    s = plain.sizes(cfg)
    assert s["hd"] == 32 and s["H"] // s["nh"] == 16
    p = "model.layers.1.self_attn."
    w = {k: v.double() for k, v in w.items()}
    w[p + "q_norm.weight"] = w[p + "q_norm.weight"] * 3.0
    w[p + "k_norm.weight"] = w[p + "k_norm.weight"] * 3.0
    torch.manual_seed(11)
    h = torch.randn(19, s["H"], dtype=torch.float64)
    positions = torch.arange(19)
    ours = plain.attention_block(h, w, p, s, positions)
    lib = _library_attention_block(h, w, p, cfg, positions)
    torch.testing.assert_close(ours, lib, rtol=1e-9, atol=1e-12)
    # what the pin catches: scores scaled by (hidden/heads)^-0.5 instead (the same as q
    # norm weights times sqrt(2) here) move the output by far more than the tolerance
    w_off = dict(w)
    w_off[p + "q_norm.weight"] = w[p + "q_norm.weight"] * ((s["H"] // s["nh"]) ** -0.5 / s["hd"] ** -0.5)
    off = plain.attention_block(h, w_off, p, s, positions)
    assert float((off - lib).abs().max()) > 1e-3 * float(lib.abs().max())


def test_qk_norms_use_the_models_eps_inside_the_root(folders):
    """Hidden states so small that the mean square of a projected head (about 1e-6)
    lies below eps (1e-5, configuration B): the per-head norms then depend on eps,
    its place and its value, by a factor of about three.  Against the library
    composition with F.rms_norm(eps=rms_norm_eps)."""
    cfg, w = folders["B"]
    s = plain.sizes(cfg)
    assert s["eps"] == 1e-5
    p = "model.layers.0.self_attn."
    w = {k: v.double() for k, v in w.items()}
    torch.manual_seed(12)
    h = torch.randn(9, s["H"], dtype=torch.float64)
    q = F.linear(h, w[p + "q_proj.weight"])
    h = h * (1e-3 / float(q.pow(2).mean().sqrt()))                 # projected heads ~ 1e-3
    positions = torch.arange(9)
    ours = plain.attention_block(h, w, p, s, positions)
    lib = _library_attention_block(h, w, p, cfg, positions)
    torch.testing.assert_close(ours, lib, rtol=1e-9, atol=1e-15)
    other = _library_attention_block(h, w, p, dict(cfg, rms_norm_eps=1e-6), positions)
    assert float((other - lib).abs().max()) > 1e-3 * float(lib.abs().max())


def test_v_is_not_normed(folders):
    """Attention is linear in v: three times v_proj gives three times the sub-layer's
    output.  A norm on v (as q and k have) would undo the factor."""
    for key in ("A", "B"):
        cfg, w = folders[key]
        s = plain.sizes(cfg)
        p = "model.layers.0.self_attn."
        w = {k: v.double() for k, v in w.items()}
        torch.manual_seed(13)
        h = torch.randn(6, s["H"], dtype=torch.float64)
        base = plain.attention_block(h, w, p, s, torch.arange(6))
        w3 = dict(w)
        w3[p + "v_proj.weight"] = w[p + "v_proj.weight"] * 3.0
        torch.testing.assert_close(plain.attention_block(h, w3, p, s, torch.arange(6)), 3.0 * base,
                                   rtol=1e-10, atol=1e-14)
        assert float(base.abs().max()) > 1e-4


def test_float64_agrees_with_float32(folders):
    cfg, w = folders["B"]
    ids = list(range(1, 40))
    w64 = {k: v.double() for k, v in w.items()}
    torch.testing.assert_close(plain.logits(ids, cfg, w), plain.logits(ids, cfg, w64), rtol=0, atol=2e-5)


# -- sampler vectors (reference tests/unit/test_sampler.py:12-56) ----------------
def test_sampler_vectors():
    p = plain.sampling_probs(torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0]), 1.0, 2, 1.0)
    assert set(torch.nonzero(p).flatten().tolist()) == {3, 4}
    p = plain.sampling_probs(torch.tensor([0.5, 0.3, 0.2]).log(), 1.0, 0, 0.7)
    assert set(torch.nonzero(p).flatten().tolist()) == {0, 1}
    torch.testing.assert_close(p[:2], torch.tensor([0.625, 0.375], dtype=torch.float64), rtol=1e-6, atol=1e-6)
    p = plain.sampling_probs(torch.tensor([0.9, 0.06, 0.04]).log(), 1.0, 0, 0.05)
    assert torch.nonzero(p).flatten().tolist() == [0]
    torch.manual_seed(0)
    logits = torch.randn(100)
    p = plain.sampling_probs(logits, 2.0, 1, 1.0)     # top_k = 1 is greedy at any temperature
    assert int(p.argmax()) == int(logits.argmax()) and p.max() == 1.0
    p = plain.sampling_probs(logits, 0.5, 0, 1.0)
    torch.testing.assert_close(p, torch.softmax(logits.double() / 0.5, -1))


def test_the_kernel_tests_own_helpers_agree_with_each_other():
    """The page packing without a loop equals the token-by-token one (written from the
    documented layout), and the blocked float64 attention equals the query-by-query one."""
    from kernel_util import pack_pages, pack_pages_whole, reference_attention, reference_attention_blocked

    g = torch.Generator().manual_seed(3)
    T, nkv, hd, ps = 77, 2, 32, 16
    k, v = torch.randn(T, nkv, hd, generator=g), torch.randn(T, nkv, hd, generator=g)
    table = [4, 0, 6, 2, 5]
    a = [torch.zeros(8, nkv * hd * ps) for _ in range(2)]
    b = [torch.zeros(8, nkv * hd * ps) for _ in range(2)]
    pack_pages(a[0], a[1], k, v, table, ps)
    pack_pages_whole(b[0], b[1], k, v, table, ps)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    q = torch.randn(9, 4, hd, generator=g)
    positions = [3, 20, 21, 40, 41, 42, 60, 75, 76]
    one = reference_attention(q, k, v, positions, 0.3)
    two = reference_attention_blocked(q, k, v, positions, 0.3, block=4)
    torch.testing.assert_close(one, two, rtol=1e-12, atol=1e-12)


def test_attention_in_blocks_of_queries_is_the_same_arithmetic(tmp_path):
    """``query_block`` only bounds memory for long sequences: the same logits."""
    folder = make_folder(tmp_path, "B")
    cfg, w = plain.read_folder(folder)
    ids = torch.randint(0, cfg["vocab_size"], (45,), generator=torch.Generator().manual_seed(1)).tolist()
    whole = plain.logits(ids, cfg, w)
    for block in (1, 7, 16, 45, 100):
        torch.testing.assert_close(plain.logits(ids, cfg, w, query_block=block), whole, rtol=0, atol=2e-6)
