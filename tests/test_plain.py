"""Pins the plain implementation by what fixes it beside the reference's text:
special cases that reduce to a library routine, invariants, and the vectors the
reference's own tests hold.  Each is chosen so that a plausible mistake (a wrong
sign or pairing, a norm in the wrong place, the gate in the wrong half) fails."""
import math

import pytest
import torch
import torch.nn.functional as F

from plain import llama_plain as P

torch.manual_seed(0)


def test_rms_norm_formula_and_scale_invariance():
    # oracle of the reference's test (tests/test_fused_ops.py:21-22), random gamma, eps 1e-5
    x, w = torch.randn(7, 256, dtype=torch.float64), torch.randn(256, dtype=torch.float64)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w
    torch.testing.assert_close(P.rms_norm(x, w, 1e-5), want)
    out = P.rms_norm(x, torch.ones(256, dtype=torch.float64), 1e-12)
    torch.testing.assert_close(out.pow(2).mean(-1), torch.ones(7, dtype=torch.float64))  # unit RMS when w = 1
    torch.testing.assert_close(P.rms_norm(3.0 * x, w, 1e-12), P.rms_norm(x, w, 1e-12))   # the scale of x drops out
    # mean of squares, not variance: a constant row keeps its sign and size
    c = torch.full((1, 8), 2.0, dtype=torch.float64)
    torch.testing.assert_close(P.rms_norm(c, torch.ones(8, dtype=torch.float64), 0.0), torch.ones(1, 8, dtype=torch.float64))


def test_swiglu_gate_is_the_first_half():
    gu = torch.randn(5, 2 * 172, dtype=torch.float64)
    torch.testing.assert_close(P.swiglu(gu), F.silu(gu[:, :172]) * gu[:, 172:])  # tests/test_fused_ops.py:71-72
    g = torch.tensor([[10.0, -10.0, 1.0, 1.0]], dtype=torch.float64)  # gate (10, -10), up (1, 1)
    out = P.swiglu(g)
    assert out[0, 0] > 9.9 and abs(out[0, 1]) < 1e-3  # swapped halves would give silu(1) * +-10


def test_mlp_uses_cat_gate_up():
    # tests/test_weight_loader.py:47-56: gate_up == cat([gate, up], 0)
    x, wg, wu, wd = torch.randn(3, 16), torch.randn(24, 16), torch.randn(24, 16), torch.randn(16, 24)
    want = (F.silu(x @ wg.T) * (x @ wu.T)) @ wd.T
    torch.testing.assert_close(P.mlp(x, wg, wu, wd), want)


def test_rope_position_zero_is_identity_and_pairs_are_half_split():
    hd = 16
    inv = P.rope_inv_freq(hd, 10000.0)
    assert inv[0] == 1.0 and torch.all(inv[1:] < inv[:-1])  # theta^0 first, then falling
    x = torch.randn(2, 3, hd, dtype=torch.float64)
    cos, sin = P.rope_cos_sin(torch.zeros(3, dtype=torch.long), inv)
    torch.testing.assert_close(P.apply_rope(x, cos, sin), x)  # the set-up of tests/test_fused_rope.py:70-85
    # a unit vector on dimension 0 at position 1 turns into (cos 1) e_0 + (sin 1) e_{hd/2}:
    # an interleaved pairing would land on e_1, a wrong sign on -sin
    e0 = torch.zeros(1, 1, hd, dtype=torch.float64)
    e0[..., 0] = 1.0
    cos, sin = P.rope_cos_sin(torch.tensor([1]), inv)
    out = P.apply_rope(e0, cos, sin)[0, 0]
    assert abs(out[0] - math.cos(1.0)) < 1e-6 and abs(out[hd // 2] - math.sin(1.0)) < 1e-6
    assert out[1].abs() < 1e-12 and out.norm() == pytest.approx(1.0, abs=1e-6)


def test_rope_scores_depend_on_distance_only():
    hd = 32
    inv = P.rope_inv_freq(hd, 500000.0)
    q, k = torch.randn(1, 1, hd, dtype=torch.float64), torch.randn(1, 1, hd, dtype=torch.float64)

    def score(m, n):
        cq, sq = P.rope_cos_sin(torch.tensor([m]), inv)
        ck, sk = P.rope_cos_sin(torch.tensor([n]), inv)
        return float((P.apply_rope(q, cq, sq) * P.apply_rope(k, ck, sk)).sum())

    assert score(7, 3) == pytest.approx(score(47, 43), abs=1e-4)
    assert score(7, 3) != pytest.approx(score(7, 4), abs=1e-3)
    # per pair the norm is kept
    cq, sq = P.rope_cos_sin(torch.tensor([11]), inv)
    r = P.apply_rope(q, cq, sq)[0, 0]
    torch.testing.assert_close(r[:16] ** 2 + r[16:] ** 2, q[0, 0, :16] ** 2 + q[0, 0, 16:] ** 2, atol=1e-6, rtol=1e-6)


def test_llama3_scaling_invariants():
    inv = P.rope_inv_freq(64, 500000.0)
    same = P.llama3_scale_inv_freq(inv, 1.0, 1.0, 4.0, 8192)
    torch.testing.assert_close(same, inv)  # factor 1 changes nothing
    out = P.llama3_scale_inv_freq(inv, 32.0, 1.0, 4.0, 8192)
    wavelen = 2 * math.pi / inv
    short, long_ = wavelen < 8192 / 4.0, wavelen > 8192 / 1.0
    assert short.any() and long_.any() and (~short & ~long_).any()
    torch.testing.assert_close(out[short], inv[short])            # short wavelengths untouched
    torch.testing.assert_close(out[long_], inv[long_] / 32.0)     # long ones divided by the factor
    assert torch.all(out[1:] <= out[:-1])                         # still falling with the index
    assert torch.all(out <= inv + 1e-12) and torch.all(out >= inv / 32.0 - 1e-12)
    # continuous at both thresholds: just inside the band equals just outside
    for wl, want_ratio in ((8192 / 4.0, 1.0), (8192 / 1.0, 1 / 32.0)):
        f = torch.tensor([2 * math.pi / (wl * 1.0001), 2 * math.pi / (wl * 0.9999)])
        r = P.llama3_scale_inv_freq(f, 32.0, 1.0, 4.0, 8192) / f
        assert r[0] == pytest.approx(want_ratio, rel=2e-3) and r[1] == pytest.approx(want_ratio, rel=2e-3)


def test_attention_reduces_to_sdpa():
    # the reference's oracle (tests/test_flash_attn.py:30-39): SDPA on repeat_interleaved K/V
    nh, nkv, S, hd = 16, 4, 24, 32
    q, k, v = (torch.randn(n, S, hd, dtype=torch.float64) for n in (nh, nkv, nkv))
    pos = torch.arange(S)
    got = P.attention(q, k, v, pos, pos)
    want = F.scaled_dot_product_attention(q[None], k.repeat_interleave(4, 0)[None], v.repeat_interleave(4, 0)[None],
                                          is_causal=True)[0]
    torch.testing.assert_close(got, want)
    # no mask: queries placed after every key see all of them
    got = P.attention(q, k, v, pos + S, pos)
    want = F.scaled_dot_product_attention(q[None], k.repeat_interleave(4, 0)[None], v.repeat_interleave(4, 0)[None])[0]
    torch.testing.assert_close(got, want)
    # as many key/value heads as query heads: plain multi-head attention
    k2, v2 = torch.randn(nh, S, hd, dtype=torch.float64), torch.randn(nh, S, hd, dtype=torch.float64)
    torch.testing.assert_close(P.attention(q, k2, v2, pos, pos),
                               F.scaled_dot_product_attention(q[None], k2[None], v2[None], is_causal=True)[0])


def test_attention_special_cases():
    hd = 16
    q, k, v = torch.randn(2, 1, hd), torch.randn(1, 1, hd), torch.randn(1, 1, hd)
    out = P.attention(q, k, v, torch.tensor([0]), torch.tensor([0]))
    torch.testing.assert_close(out, v.expand(2, 1, hd))  # one key: the output is its value
    # grouped heads: query heads 0,1 read key/value head 0 and 2,3 read head 1 (h // g, not h % nkv)
    q = torch.zeros(4, 1, hd)
    k = torch.zeros(2, 3, hd)
    v = torch.stack([torch.full((3, hd), 1.0), torch.full((3, hd), 2.0)])
    out = P.attention(q, k, v, torch.tensor([2]), torch.arange(3))
    assert out[:2].eq(1.0).all() and out[2:].eq(2.0).all()
    # a query in the middle of a sequence sees the keys before it (absolute positions)
    q, k, v = torch.randn(1, 2, hd), torch.randn(1, 6, hd), torch.randn(1, 6, hd)
    part = P.attention(q, k, v, torch.tensor([4, 5]), torch.arange(6))
    whole = P.attention(torch.cat([torch.randn(1, 4, hd), q], 1), k, v, torch.arange(6), torch.arange(6))
    torch.testing.assert_close(part, whole[:, 4:])
    # a window of 2: position 5 sees keys 4 and 5 only
    w = P.attention(q[:, 1:], k, v, torch.tensor([5]), torch.arange(6), window=2)
    torch.testing.assert_close(w, P.attention(q[:, 1:], k[:, 4:], v[:, 4:], torch.tensor([5]), torch.tensor([4, 5])))


def tiny_weights(cfg, seed=0, std=0.1):
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    w = {"model.embed_tokens.weight": torch.randn(V, H, generator=g) * std,
         "model.norm.weight": 1 + 0.1 * torch.randn(H, generator=g)}
    if not cfg.get("tie_word_embeddings"):
        w["lm_head.weight"] = torch.randn(V, H, generator=g) * std
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g)
        for n, shape in (("self_attn.q_proj", (nh * hd, H)), ("self_attn.k_proj", (nkv * hd, H)),
                         ("self_attn.v_proj", (nkv * hd, H)), ("self_attn.o_proj", (H, nh * hd)),
                         ("mlp.gate_proj", (I, H)), ("mlp.up_proj", (I, H)), ("mlp.down_proj", (H, I))):
            w[p + n + ".weight"] = torch.randn(*shape, generator=g) * std
    return w


CFG = dict(vocab_size=50, hidden_size=32, intermediate_size=40, num_hidden_layers=2, num_attention_heads=4,
           num_key_value_heads=2, head_dim=8, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False)


def test_forward_is_causal_and_a_prefix_is_enough():
    w = tiny_weights(CFG)
    toks = [3, 14, 15, 9, 26, 5, 35]
    full = P.forward(w, CFG, toks)
    torch.testing.assert_close(P.forward(w, CFG, toks[:4]), full[:4])       # later tokens do not reach back
    changed = P.forward(w, CFG, toks[:6] + [1])
    torch.testing.assert_close(changed[:6], full[:6])
    assert not torch.allclose(changed[6], full[6])


def test_forward_tied_head_equals_copied_matrix():
    # the reference copies the embedding into lm_head when the file has none (weight_loader.py:106-109)
    w = tiny_weights(dict(CFG, tie_word_embeddings=True))
    tied = P.forward(w, dict(CFG, tie_word_embeddings=True), [1, 2, 3])
    w2 = dict(w, **{"lm_head.weight": w["model.embed_tokens.weight"].clone()})
    torch.testing.assert_close(tied, P.forward(w2, CFG, [1, 2, 3]))


def test_forward_norm_placement_and_residuals():
    """Zero projections out of the mixer and the feed-forward: the model is
    embed -> final norm -> head, which pins the final norm and shows that both
    branches only ever add to the stream."""
    w = tiny_weights(CFG)
    for k in w:
        if k.endswith("o_proj.weight") or k.endswith("down_proj.weight"):
            w[k] = torch.zeros_like(w[k])
    toks = [7, 8, 9]
    e = w["model.embed_tokens.weight"][torch.tensor(toks)].double()
    want = P.rms_norm(e, w["model.norm.weight"].double(), CFG["rms_norm_eps"]) @ w["lm_head.weight"].double().T
    torch.testing.assert_close(P.forward(w, CFG, toks), want)


def test_rope_frequencies_elementwise():
    """theta^(-2i/d) for i = 0 .. d/2 - 1, as models/llama.py:180-183 and the oracle of
    tests/test_fused_rope.py:16-18 (arange(0, d, 2) / d): an exponent of i/d would pass
    "first is 1, then falling" and fails here."""
    for d, theta in ((16, 10000.0), (64, 500000.0), (128, 10000.0)):
        inv = P.rope_inv_freq(d, theta)
        assert inv.shape == (d // 2,)
        want = torch.tensor([theta ** (-2.0 * i / d) for i in range(d // 2)], dtype=torch.float64)
        torch.testing.assert_close(inv.double(), want, rtol=1e-6, atol=0)
        assert float(inv[-1]) == pytest.approx(theta ** (-(d - 2) / d), rel=1e-6)   # the slowest pair: almost 1/theta
    # the table's angle at position p is p * inv_freq: the pair (i, i + d/2) of a one-hot vector turns by it
    inv = P.rope_inv_freq(8, 100.0)
    e = torch.zeros(1, 1, 8, dtype=torch.float64)
    e[..., 2] = 1.0
    cos, sin = P.rope_cos_sin(torch.tensor([5]), inv)
    out = P.apply_rope(e, cos, sin)[0, 0]
    angle = 5 * 100.0 ** (-2.0 * 2 / 8)
    assert abs(out[2] - math.cos(angle)) < 1e-6 and abs(out[6] - math.sin(angle)) < 1e-6


def test_llama3_middle_band_is_a_straight_blend():
    """Inside the band the new frequency is (1 - s) f / factor + s f with s running straight from 0
    at wavelength L / low to 1 at L / high in L / wavelength: halfway it is the mean of the two ends,
    a quarter in it is 3:1.  Continuity at the ends alone would also pass a curve of another shape."""
    L, low, high, factor = 8192.0, 1.0, 4.0, 32.0
    for s in (0.25, 0.5, 0.75):
        ratio = low + s * (high - low)            # L / wavelength
        f = torch.tensor([2 * math.pi * ratio / L], dtype=torch.float64)
        out = P.llama3_scale_inv_freq(f, factor, low, high, L)
        want = (1 - s) * f / factor + s * f
        torch.testing.assert_close(out.double(), want, rtol=1e-6, atol=0)


def test_each_norm_stands_before_its_own_branch():
    """A norm weight of zero silences the branch behind it and nothing else (no biases anywhere):
    with input_layernorm = 0 the layer is h + mlp(norm2(h)), with post_attention_layernorm = 0 it is
    h + attention(norm1(h)).  Swapped norm weights, a norm after the branch, or a branch fed from
    the wrong stream fail one of the two (models/llama.py:147-165)."""
    cfg = dict(CFG, num_hidden_layers=1)
    w = {k: v.double() for k, v in tiny_weights(cfg, seed=3).items()}
    p = "model.layers.0."
    S = 5
    h = torch.randn(S, cfg["hidden_size"], dtype=torch.float64)
    pos = torch.arange(S)
    inv = P.model_inv_freq(cfg)
    eps = cfg["rms_norm_eps"]

    w1 = dict(w, **{p + "input_layernorm.weight": torch.zeros_like(w[p + "input_layernorm.weight"])})
    want = h + P.mlp(P.rms_norm(h, w[p + "post_attention_layernorm.weight"], eps), w[p + "mlp.gate_proj.weight"],
                     w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    torch.testing.assert_close(P.decoder_layer(h, pos, w1, 0, cfg, inv), want)

    w2 = dict(w, **{p + "post_attention_layernorm.weight": torch.zeros_like(w[p + "input_layernorm.weight"])})
    x = P.rms_norm(h, w[p + "input_layernorm.weight"], eps)
    want = h + P.attention_layer(x, pos, w, p + "self_attn.", cfg, inv)
    torch.testing.assert_close(P.decoder_layer(h, pos, w2, 0, cfg, inv), want)
    # the second branch reads the stream *after* the first was added: with both norms alive the
    # result differs from the sum of the two single-branch results
    both = P.decoder_layer(h, pos, w, 0, cfg, inv)
    alone = P.decoder_layer(h, pos, w1, 0, cfg, inv) + P.decoder_layer(h, pos, w2, 0, cfg, inv) - h
    assert not torch.allclose(both, alone, atol=1e-6)
    h1 = h + P.attention_layer(x, pos, w, p + "self_attn.", cfg, inv)
    want = h1 + P.mlp(P.rms_norm(h1, w[p + "post_attention_layernorm.weight"], eps), w[p + "mlp.gate_proj.weight"],
                      w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    torch.testing.assert_close(both, want)


def test_sampling_follows_the_reference_rules():
    logits = torch.tensor([2.0, 1.0, 0.5, 0.0, -1.0, -3.0])
    assert P.greedy(logits) == 0
    p = P.sample_filter(logits, 0.7, top_k=1, top_p=1.0)
    assert p[0] == 1.0                                             # top-k 1 is greedy
    p = P.sample_filter(logits, 1.0, top_k=3, top_p=1.0)
    assert (p[:3] > 0).all() and (p[3:] == 0).all()
    torch.testing.assert_close(p[:3], torch.softmax(logits[:3].double(), 0))
    # top-p: probabilities 0.574 0.211 0.128 ...; p = 0.6 keeps the token that crosses 0.6 (the second)
    p = P.sample_filter(logits, 1.0, top_k=-1, top_p=0.6)
    assert (p[:2] > 0).all() and (p[2:] == 0).all()
    p = P.sample_filter(logits, 1.0, top_k=-1, top_p=0.0)
    assert p[0] == 1.0                                             # the first is never removed
    cold = P.sample_filter(logits, 0.01, -1, 1.0)
    assert cold[0] > 0.999                                         # T -> 0 tends to the argmax
    probs = torch.tensor([0.1, 0.2, 0.3, 0.4])
    assert [P.inverse_cdf(probs, u) for u in (0.0, 0.05, 0.1, 0.29, 0.3, 0.95, 0.9999)] == [0, 0, 1, 1, 2, 3, 3]


def test_the_long_request_helper_is_the_plain_forward(tmp_path):
    """``trace_util.plain_logits_at`` (queries a few at a time, the last layer at the wanted places
    only) gives what ``P.forward`` gives."""
    import json
    import os

    from safetensors.torch import save_file
    from trace_util import plain_logits_at

    cfg = dict(CFG, num_hidden_layers=3, rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                                                           high_freq_factor=4.0, original_max_position_embeddings=16))
    w = tiny_weights(cfg, seed=5)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(tmp_path, "model.safetensors"))
    json.dump(cfg, open(os.path.join(tmp_path, "config.json"), "w"))
    toks = torch.randint(0, cfg["vocab_size"], (41,), generator=torch.Generator().manual_seed(1)).tolist()
    w2, cfg2 = P.read_model(str(tmp_path))
    full = P.forward(w2, cfg2, toks)
    got = plain_logits_at(str(tmp_path), toks, [40, 0, 17, 39], chunk=7)
    assert sorted(got) == [0, 17, 39, 40]
    for r, row in got.items():
        torch.testing.assert_close(row, full[r], rtol=1e-9, atol=1e-9)
