"""Pins of the plain implementation by what fixes it beside the reference's text: library
routines it must reduce to, invariants, and the vectors the reference's own files hold.
Each check is chosen so that a plausible mistake fails it."""
import math

import torch
import torch.nn.functional as F

import plain_qwen2 as plain

torch.manual_seed(0)


def test_rms_norm_is_the_library_routine():
    x = torch.randn(5, 96, dtype=torch.float64)
    w = torch.randn(96, dtype=torch.float64)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5))


def test_rms_norm_eps_inside_root_and_weight_last():
    # a zero row stays zero (eps outside the root would divide by zero)
    assert torch.equal(plain.rms_norm(torch.zeros(2, 8, dtype=torch.float64), torch.ones(8, dtype=torch.float64), 1e-6),
                       torch.zeros(2, 8, dtype=torch.float64))
    # weight 1 and tiny eps: unit mean square; a (1 + w) offset would double it
    y = plain.rms_norm(torch.randn(3, 64, dtype=torch.float64) * 7, torch.ones(64, dtype=torch.float64), 1e-12)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(3, dtype=torch.float64))
    # scale invariance of the input
    x = torch.randn(3, 64, dtype=torch.float64)
    w = torch.randn(64, dtype=torch.float64)
    torch.testing.assert_close(plain.rms_norm(5 * x, w, 1e-12), plain.rms_norm(x, w, 1e-12))
    # eps matters as an addend to the mean square, not to the root
    x = torch.full((1, 4), 2.0, dtype=torch.float64)
    torch.testing.assert_close(plain.rms_norm(x, torch.ones(4, dtype=torch.float64), 5.0), x / 3.0)


def test_linear_is_the_library_routine():
    x, w, b = torch.randn(4, 7, dtype=torch.float64), torch.randn(5, 7, dtype=torch.float64), torch.randn(5, dtype=torch.float64)
    torch.testing.assert_close(plain.linear(x, w, b), F.linear(x, w, b))


def test_rope_reference_self_check_vector():
    """The reference's own check (v00_full_recompute/layer/rope.py:77-100): seed 42, x of
    shape (2,4,8,64), theta 1e4: the rotation keeps the shape and every vector's norm to 1e-5."""
    torch.manual_seed(42)
    x = torch.randn(2, 4, 8, 64)
    y = torch.stack([plain.rope_apply(x[b], torch.arange(8), 10000.0) for b in range(2)])
    assert y.shape == x.shape
    assert torch.allclose(torch.norm(x.float(), dim=-1), torch.norm(y.float(), dim=-1), atol=1e-5)


def test_rope_position_zero_is_identity_and_pairs_are_split_half():
    x = torch.randn(3, 1, 16, dtype=torch.float64)
    torch.testing.assert_close(plain.rope_apply(x, torch.tensor([0]), 1e4), x)
    # one-hot at feature 0 and position 1: the partner is feature hd/2, not feature 1
    e = torch.zeros(1, 1, 16, dtype=torch.float64)
    e[0, 0, 0] = 1.0
    y = plain.rope_apply(e, torch.tensor([1]), 1e4)[0, 0]
    assert abs(float(y[0]) - math.cos(1.0)) < 1e-6 and abs(float(y[8]) - math.sin(1.0)) < 1e-6
    assert float(y[1]) == 0.0
    # the sign: rotating feature hd/2 gives -sin on feature 0
    e = torch.zeros(1, 1, 16, dtype=torch.float64)
    e[0, 0, 8] = 1.0
    y = plain.rope_apply(e, torch.tensor([1]), 1e4)[0, 0]
    assert abs(float(y[0]) + math.sin(1.0)) < 1e-6 and abs(float(y[8]) - math.cos(1.0)) < 1e-6
    # frequency j is theta ** (-2j/hd): feature 1 of a 4-wide head at position 1 turns by theta**-0.5
    e = torch.zeros(1, 1, 4, dtype=torch.float64)
    e[0, 0, 1] = 1.0
    y = plain.rope_apply(e, torch.tensor([1]), 100.0)[0, 0]
    assert abs(float(y[1]) - math.cos(0.1)) < 1e-6 and abs(float(y[3]) - math.sin(0.1)) < 1e-6


def test_rope_scores_depend_on_distance_only():
    q, k = torch.randn(1, 1, 32, dtype=torch.float64), torch.randn(1, 1, 32, dtype=torch.float64)
    def score(m, n):
        return float((plain.rope_apply(q, torch.tensor([m]), 1e4) * plain.rope_apply(k, torch.tensor([n]), 1e4)).sum())
    assert abs(score(9, 4) - score(25, 20)) < 1e-5      # float32 angles: equal to rounding
    assert abs(score(9, 4) - score(9, 5)) > 1e-3


def test_attention_without_rotation_is_library_attention():
    heads, kvh, t, hd = 6, 2, 11, 16
    q, k, v = (torch.randn(n, t, hd, dtype=torch.float64) for n in (heads, kvh, kvh))
    w = plain.attention_weights(q, k.repeat_interleave(3, 0))
    got = w @ v.repeat_interleave(3, 0)
    ref = F.scaled_dot_product_attention(q[None], k.repeat_interleave(3, 0)[None], v.repeat_interleave(3, 0)[None], is_causal=True)[0]
    torch.testing.assert_close(got, ref)
    torch.testing.assert_close(w.sum(-1), torch.ones(heads, t, dtype=torch.float64))
    assert float(w.triu(1).abs().max()) == 0.0


def test_attention_window_definition():
    q = k = torch.zeros(1, 6, 4, dtype=torch.float64)
    w = plain.attention_weights(q, k, window=3)[0]
    expect = torch.tensor([[1, 0, 0, 0, 0, 0], [.5, .5, 0, 0, 0, 0], [1/3, 1/3, 1/3, 0, 0, 0], [0, 1/3, 1/3, 1/3, 0, 0],
                           [0, 0, 1/3, 1/3, 1/3, 0], [0, 0, 0, 1/3, 1/3, 1/3]], dtype=torch.float64)
    torch.testing.assert_close(w, expect)


def test_attention_window_invariants_and_the_library_routine_with_a_band_mask():
    """The window is not in the reference; what fixes it here besides its definition: a window at least as
    long as the sequence is causal attention (the library routine), a window of one returns every token's
    own value, and any window equals the library routine under a band mask built from ``tril``/``triu``
    (keys ``t - W < s <= t``: a mistake by one at either edge fails it)."""
    heads, t, hd = 3, 23, 8
    q, k, v = (torch.randn(heads, t, hd, dtype=torch.float64) for _ in range(3))
    causal = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    for window in (t, t + 5):
        torch.testing.assert_close(plain.attention_weights(q, k, window=window) @ v, causal)
    torch.testing.assert_close(plain.attention_weights(q, k, window=1) @ v, v)
    for window in (2, 7, 22):
        ones = torch.ones(t, t, dtype=torch.bool)
        band = torch.tril(ones) & torch.triu(ones, diagonal=-(window - 1))
        ref = F.scaled_dot_product_attention(q[None], k[None], v[None], attn_mask=band)[0]
        torch.testing.assert_close(plain.attention_weights(q, k, window=window) @ v, ref)
        assert int(plain.attention_weights(q, k, window=window)[0].gt(0).sum(-1).max()) == window


def test_which_layers_have_a_window():
    base = dict(vocab_size=8, hidden_size=8, num_hidden_layers=5, num_attention_heads=2, intermediate_size=8)
    on = plain.PlainConfig(dict(base, use_sliding_window=True, sliding_window=9, max_window_layers=2))
    assert [on.window_of(i) for i in range(5)] == [None, None, 9, 9, 9]        # layers from max_window_layers on
    assert [plain.PlainConfig(dict(base, sliding_window=9, max_window_layers=2)).window_of(i) for i in range(5)] == [None] * 5
    assert [plain.PlainConfig(dict(base, use_sliding_window=True, sliding_window=9)).window_of(i) for i in range(5)] == [None] * 5


def _attn_weights(hidden, heads, kvh, hd, bias=True):
    w = {"q_proj.weight": torch.randn(heads * hd, hidden, dtype=torch.float64) * 0.2,
         "k_proj.weight": torch.randn(kvh * hd, hidden, dtype=torch.float64) * 0.2,
         "v_proj.weight": torch.randn(kvh * hd, hidden, dtype=torch.float64) * 0.2,
         "o_proj.weight": torch.randn(hidden, heads * hd, dtype=torch.float64) * 0.2}
    if bias:
        for n, width in (("q", heads * hd), ("k", kvh * hd), ("v", kvh * hd)):
            w[f"{n}_proj.bias"] = torch.randn(width, dtype=torch.float64) * 0.2
    return w


def test_gqa_one_token_returns_its_value_and_heads_map_to_groups():
    hidden, heads, kvh, hd = 24, 4, 2, 8
    w = _attn_weights(hidden, heads, kvh, hd)
    h = torch.randn(1, hidden, dtype=torch.float64)
    out = plain.gqa_attention(h, w, num_heads=heads, num_kv_heads=kvh, head_dim=hd, theta=1e4, positions=torch.tensor([0]))
    v = plain.linear(h, w["v_proj.weight"], w["v_proj.bias"]).view(kvh, hd)
    ctx = v.repeat_interleave(2, 0).reshape(1, -1)          # query heads 0,1 -> KV head 0; 2,3 -> KV head 1
    torch.testing.assert_close(out, plain.linear(ctx, w["o_proj.weight"]))


def test_gqa_with_equal_heads_is_multi_head_attention_and_shift_invariant():
    hidden, heads, hd, t = 32, 4, 8, 9
    w = _attn_weights(hidden, heads, heads, hd, bias=False)
    h = torch.randn(t, hidden, dtype=torch.float64)
    kw = dict(num_heads=heads, num_kv_heads=heads, head_dim=hd, theta=1e4)
    a = plain.gqa_attention(h, w, positions=torch.arange(t), **kw)
    b = plain.gqa_attention(h, w, positions=torch.arange(t) + 37, **kw)
    torch.testing.assert_close(a, b, atol=1e-5, rtol=1e-5)       # only distances count
    # last row equals attention of the last query over all keys (what decoding computes)
    q = plain.rope_apply(plain.linear(h, w["q_proj.weight"]).view(t, heads, hd).transpose(0, 1), torch.arange(t), 1e4)
    k = plain.rope_apply(plain.linear(h, w["k_proj.weight"]).view(t, heads, hd).transpose(0, 1), torch.arange(t), 1e4)
    v = plain.linear(h, w["v_proj.weight"]).view(t, heads, hd).transpose(0, 1)
    s = torch.softmax((q[:, -1:] @ k.transpose(1, 2)) / math.sqrt(hd), -1)
    last = (s @ v).transpose(0, 1).reshape(1, -1)
    torch.testing.assert_close(a[-1:], plain.linear(last, w["o_proj.weight"]))


def test_swiglu_is_silu_gate_times_up():
    w = {"gate_proj.weight": torch.randn(10, 6, dtype=torch.float64), "up_proj.weight": torch.randn(10, 6, dtype=torch.float64),
         "down_proj.weight": torch.randn(6, 10, dtype=torch.float64)}
    h = torch.randn(3, 6, dtype=torch.float64)
    g, u = h @ w["gate_proj.weight"].T, h @ w["up_proj.weight"].T
    torch.testing.assert_close(plain.swiglu_ffn(h, w), (g * torch.sigmoid(g) * u) @ w["down_proj.weight"].T)


def test_forward_tied_head_shift_and_causality(model_folders):
    cfg, w = plain.load_folder(model_folders["A"])
    assert cfg.tied and "lm_head.weight" not in w
    ids = [3, 200, 17, 5, 99, 42, 7]
    full = plain.forward(cfg, w, ids)
    assert full.shape == (7, cfg.vocab)
    # untying with a copy of the embedding gives the same logits
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    cfg2 = plain.PlainConfig({**_cfg_dict(model_folders["A"]), "tie_word_embeddings": False})
    torch.testing.assert_close(plain.forward(cfg2, w2, ids), full)
    # causal: a prefix gives the same logits at its positions
    torch.testing.assert_close(plain.forward(cfg, w, ids[:4]), full[:4], atol=1e-12, rtol=1e-9)
    # shifting every position changes nothing but rounding of the float32 angles
    torch.testing.assert_close(plain.forward(cfg, w, ids, first_position=50), full, atol=1e-6, rtol=1e-5)


def test_greedy_loop_and_stop(model_folders):
    cfg, w = plain.load_folder(model_folders["A"])
    out = plain.greedy(cfg, w, [1, 2, 3], 5)
    assert len(out) == 5
    stop = out[2]
    assert plain.greedy(cfg, w, [1, 2, 3], 5, stop_ids={stop}) == out[:out.index(stop)]


def _cfg_dict(folder):
    import json
    return json.loads((folder / "config.json").read_text())
