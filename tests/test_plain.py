"""Pins of the plain implementation by what fixes it beside the reference's text.

Each test is chosen so that a plausible mistake fails it: a wrong sign or pairing
in the rotation, a norm weight in the wrong place, a scale before instead of
after, an off-by-one at the window's edge, kv heads repeated in the wrong order.
The reference's own tests compare against a library model that is not a source
here, and its result files hold only summaries of runs with real weights, so a
whole-model vector is "parity unpinned"; the parts are pinned one by one.
"""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen2 as plain

torch.manual_seed(0)


def test_rms_norm_matches_fp64_formula_and_ignores_scale():
    x = torch.randn(5, 48, dtype=torch.float64)
    w = torch.randn(48, dtype=torch.float64)
    eps = 1e-6
    want = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w
    assert torch.allclose(plain.rms_norm(x, w, eps), want, atol=1e-12)
    # mean square of the output with weight 1 is var / (var + eps)
    y = plain.rms_norm(x, torch.ones(48, dtype=torch.float64), eps)
    var = (x * x).mean(-1)
    assert torch.allclose((y * y).mean(-1), var / (var + eps), atol=1e-12)
    # a large common factor leaves the output unchanged up to eps
    assert torch.allclose(plain.rms_norm(1e3 * x, w, eps), plain.rms_norm(x, w, eps), atol=1e-9)


def test_rms_norm_eps_is_inside_the_root():
    x = torch.full((1, 4), 2.0, dtype=torch.float64)
    y = plain.rms_norm(x, torch.ones(4, dtype=torch.float64), 5.0)
    assert torch.allclose(y, torch.full((1, 4), 2.0 / 3.0, dtype=torch.float64))


def test_inv_freq_values():
    inv = plain.rope_inv_freq(8, 10000.0, torch.float64)
    assert inv[0].item() == 1.0
    for i in range(4):
        assert math.isclose(inv[i].item(), 10000.0 ** (-2 * i / 8), rel_tol=1e-12)


def test_rope_pairing_and_sign():
    # D = 2: the pair is (0, 1); a unit vector on the first axis turns to (cos p, sin p).
    pos = torch.tensor([0, 1, 3])
    cos, sin = plain.rope_cos_sin(pos, 2, 10000.0, torch.float64, torch.float64)
    x = torch.tensor([1.0, 0.0], dtype=torch.float64).expand(3, 1, 2)
    y = plain.apply_rope(x, cos, sin)
    for t, p in enumerate([0.0, 1.0, 3.0]):
        assert torch.allclose(y[t, 0], torch.tensor([math.cos(p), math.sin(p)], dtype=torch.float64))
    # D = 4: element j pairs with j + D/2, not with j + 1.
    cos, sin = plain.rope_cos_sin(torch.tensor([2]), 4, 100.0, torch.float64, torch.float64)
    x = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]], dtype=torch.float64)
    y = plain.apply_rope(x, cos, sin)[0, 0]
    assert torch.allclose(y, torch.tensor([math.cos(2.0), 0.0, math.sin(2.0), 0.0], dtype=torch.float64))
    x = torch.tensor([[[0.0, 1.0, 0.0, 0.0]]], dtype=torch.float64)
    y = plain.apply_rope(x, cos, sin)[0, 0]
    a = 2.0 * 100.0 ** (-0.5)
    assert torch.allclose(y, torch.tensor([0.0, math.cos(a), 0.0, math.sin(a)], dtype=torch.float64))


def test_rope_identity_at_zero_norms_and_relative_scores():
    d = 16
    q = torch.randn(6, 2, d, dtype=torch.float64)
    k = torch.randn(6, 2, d, dtype=torch.float64)
    cos0, sin0 = plain.rope_cos_sin(torch.zeros(6, dtype=torch.long), d, 1e4, torch.float64, torch.float64)
    assert torch.allclose(plain.apply_rope(q, cos0, sin0), q)
    pos = torch.tensor([0, 3, 4, 9, 20, 21])
    cos, sin = plain.rope_cos_sin(pos, d, 1e4, torch.float64, torch.float64)
    rq = plain.apply_rope(q, cos, sin)
    pair = lambda x: x[..., : d // 2] ** 2 + x[..., d // 2:] ** 2
    assert torch.allclose(pair(rq), pair(q))
    cos2, sin2 = plain.rope_cos_sin(pos + 37, d, 1e4, torch.float64, torch.float64)
    s1 = torch.einsum("qhd,khd->hqk", rq, plain.apply_rope(k, cos, sin))
    s2 = torch.einsum("qhd,khd->hqk", plain.apply_rope(q, cos2, sin2), plain.apply_rope(k, cos2, sin2))
    assert torch.allclose(s1, s2, atol=1e-9)


def test_rope_angles_are_float32_as_in_the_reference():
    """worker/src/inference/qwen2/model.py:98-105 computes frequencies, angles and trigonometry in
    float32: far from position 0 that is visibly not the exact angle, and it is what the model uses."""
    pos = torch.tensor([0, 1, 2000, 4000])
    cos32, sin32 = plain.rope_cos_sin(pos, 64, 1e6, torch.float64)
    cos64, sin64 = plain.rope_cos_sin(pos, 64, 1e6, torch.float64, torch.float64)
    assert cos32.dtype == torch.float64
    assert torch.equal(cos32[0], cos64[0]) and (cos32[1] - cos64[1]).abs().max() < 1e-6
    far = (sin32[2:] - sin64[2:]).abs().max().item()
    assert 1e-6 < far < 5e-4
    freqs = pos.to(torch.float32)[:, None] * plain.rope_inv_freq(64, 1e6, torch.float32)[None, :]
    assert torch.equal(cos32[:, :32], freqs.cos().double())


def test_attention_is_library_causal_attention_when_heads_are_not_grouped():
    t, h, d = 9, 3, 8
    q, k, v = (torch.randn(t, h, d, dtype=torch.float64) for _ in range(3))
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                          v.transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(plain.attention(q, k, v), want, atol=1e-12)


def test_attention_first_token_and_window_edges():
    t, h, kh, d = 12, 4, 2, 8
    q = torch.randn(t, h, d, dtype=torch.float64)
    k = torch.randn(t, kh, d, dtype=torch.float64)
    v = torch.randn(t, kh, d, dtype=torch.float64)
    out = plain.attention(q, k, v)
    # the first token sees only itself: its output is its own value, per kv head
    assert torch.allclose(out[0], plain.repeat_kv(v, 2)[0])
    # a window as long as the sequence changes nothing; a window of 1 gives every token its own value
    assert torch.allclose(plain.attention(q, k, v, window=t), out)
    assert torch.allclose(plain.attention(q, k, v, window=1), plain.repeat_kv(v, 2))
    # window w: exactly the keys i-w+1..i count. Brute force for one query.
    w = 5
    got = plain.attention(q, k, v, window=w)
    i, head = 9, 3
    keys = range(i - w + 1, i + 1)
    s = torch.stack([(q[i, head] * k[j, head // 2]).sum() / math.sqrt(d) for j in keys])
    p = torch.softmax(s, 0)
    want = sum(p[n] * v[j, head // 2] for n, j in enumerate(keys))
    assert torch.allclose(got[i, head], want, atol=1e-12)
    assert plain.visibility(12, 5)[9].nonzero().flatten().tolist() == [5, 6, 7, 8, 9]


def test_grouped_heads_read_kv_head_h_div_g():
    t, h, kh, d = 5, 6, 2, 4
    q = torch.randn(t, h, d, dtype=torch.float64)
    k = torch.randn(t, kh, d, dtype=torch.float64)
    v = torch.randn(t, kh, d, dtype=torch.float64)
    out = plain.attention(q, k, v)
    for head in range(h):
        alone = plain.attention(q[:, head:head + 1], k[:, head // 3:head // 3 + 1], v[:, head // 3:head // 3 + 1])
        assert torch.allclose(out[:, head:head + 1], alone, atol=1e-12)


def test_scale_is_head_dim_to_minus_half():
    q = torch.tensor([[[2.0, 0.0, 0.0, 0.0]], [[2.0, 0.0, 0.0, 0.0]]], dtype=torch.float64)
    k = torch.tensor([[[0.0, 0, 0, 0]], [[3.0, 0, 0, 0]]], dtype=torch.float64)
    v = torch.tensor([[[1.0, 0, 0, 0]], [[0.0, 1, 0, 0]]], dtype=torch.float64)
    out = plain.attention(q, k, v)
    p = math.exp(3.0) / (1 + math.exp(3.0))  # score 6 * 4^-0.5 = 3
    assert torch.allclose(out[1, 0, :2], torch.tensor([1 - p, p], dtype=torch.float64))


def test_swiglu_reductions():
    x = torch.randn(4, 10, dtype=torch.float64)
    assert torch.allclose(plain.silu(x), F.silu(x), atol=1e-12)
    wg = torch.randn(7, 10, dtype=torch.float64)
    wd = torch.randn(10, 7, dtype=torch.float64)
    wu = torch.zeros(7, 10, dtype=torch.float64)
    x1 = x.clone()
    x1[:, 0] = 1.0
    wu[:, 0] = 1.0  # up(x) == 1
    wg[:, 0] = 0.0
    assert torch.allclose(plain.swiglu(x1, wg, wu, wd), F.silu(x1 @ wg.T) @ wd.T, atol=1e-12)


@pytest.mark.parametrize("cfg", [plain.TINY_A, plain.TINY_B, plain.TINY_C])
def test_shift_of_all_positions_changes_nothing(cfg):
    w = plain.random_weights(cfg, 1, std=0.3, norm_jitter=0.2)
    ids = torch.randint(0, cfg["vocab_size"], (30,), generator=torch.Generator().manual_seed(2))
    # with exact angles only distances count; with the reference's float32 angles (the default) nearly
    a = plain.forward(w, cfg, ids, torch.float64, angle_dtype=torch.float64)
    b = plain.forward(w, cfg, ids, torch.float64, first_position=41, angle_dtype=torch.float64)
    assert torch.allclose(a, b, atol=1e-8)
    assert a.shape == (30, cfg["vocab_size"])
    c = plain.forward(w, cfg, ids, torch.float64, first_position=41)
    assert torch.allclose(a, c, atol=1e-3) and not torch.allclose(a, c, atol=1e-9)


def test_logits_are_causal_and_windows_follow_the_config():
    cfg = plain.TINY_B
    assert plain.layer_windows(cfg) == [None, 8, 8]
    assert plain.layer_windows(plain.TINY_A) == [None, None]
    assert plain.layer_windows(plain.TINY_C) == [20, None]
    w = plain.random_weights(cfg, 3, std=0.3)
    ids = torch.randint(0, cfg["vocab_size"], (25,), generator=torch.Generator().manual_seed(4))
    full = plain.forward(w, cfg, ids, torch.float64)
    part = plain.forward(w, cfg, ids[:11], torch.float64)
    assert torch.allclose(full[:11], part, atol=1e-9)
    # with the window switched off the late logits differ: the window is really applied
    off = dict(cfg, use_sliding_window=False)
    assert not torch.allclose(plain.forward(w, off, ids, torch.float64)[-1], full[-1], atol=1e-6)
    assert torch.allclose(plain.forward(w, off, ids, torch.float64)[:8], full[:8], atol=1e-9)


def test_tied_head_is_the_embedding():
    cfg = plain.TINY_A
    w = plain.random_weights(cfg, 5, std=0.3)
    assert "lm_head.weight" not in w
    ids = [3, 1, 4]
    logits = plain.forward(w, cfg, ids, torch.float64)
    untied = dict(cfg, tie_word_embeddings=False)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    assert torch.allclose(plain.forward(w2, untied, ids, torch.float64), logits)


def test_one_layer_one_head_by_hand():
    """The whole block, spelled out with library routines for one head."""
    cfg = dict(plain.TINY_A, num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1,
               hidden_size=16, intermediate_size=24, vocab_size=50)
    w = plain.random_weights(cfg, 6, std=0.4, norm_jitter=0.3, dtype=torch.float64)
    ids = torch.tensor([7, 8, 9, 3, 3])
    x = w["model.embed_tokens.weight"][ids]
    p = "model.layers.0."
    rms = lambda t, g: t / torch.sqrt((t * t).mean(-1, keepdim=True) + 1e-6) * g
    n = rms(x, w[p + "input_layernorm.weight"])
    q = n @ w[p + "self_attn.q_proj.weight"].T + w[p + "self_attn.q_proj.bias"]
    k = n @ w[p + "self_attn.k_proj.weight"].T + w[p + "self_attn.k_proj.bias"]
    v = n @ w[p + "self_attn.v_proj.weight"].T + w[p + "self_attn.v_proj.bias"]
    ang = torch.arange(5, dtype=torch.float64)[:, None] * (10000.0 ** (-torch.arange(8, dtype=torch.float64) / 8))[None]
    def rot(t):
        a, b = t[:, :8], t[:, 8:]
        return torch.cat([a * ang.cos() - b * ang.sin(), b * ang.cos() + a * ang.sin()], -1)
    att = F.scaled_dot_product_attention(rot(q)[None], rot(k)[None], v[None], is_causal=True)[0]
    x = x + att @ w[p + "self_attn.o_proj.weight"].T
    n = rms(x, w[p + "post_attention_layernorm.weight"])
    x = x + (F.silu(n @ w[p + "mlp.gate_proj.weight"].T) * (n @ w[p + "mlp.up_proj.weight"].T)) @ w[p + "mlp.down_proj.weight"].T
    want = rms(x, w["model.norm.weight"]) @ w["model.embed_tokens.weight"].T
    assert torch.allclose(plain.forward(w, cfg, ids, torch.float64), want, atol=1e-10)
