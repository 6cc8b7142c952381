"""Pins the plain implementation by what fixes it beside the reference's text: special cases that
reduce to a library routine, closed forms and invariants, each chosen so that a plausible
mistake (a wrong sign or pairing, a norm or a scale in the wrong place) fails it.  No GPU."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_model as pm
from conftest import TINY

torch.manual_seed(0)
D = torch.float64


def rand(*shape):
    return torch.randn(*shape, dtype=D)


# ---- RMSNorm ------------------------------------------------------------------------------
def test_rms_norm_closed_form_and_eps_inside_the_root():
    c, eps = 3.0, 1e-6
    y = pm.rms_norm(torch.full((2, 8), c, dtype=D), torch.ones(8, dtype=D), eps)
    assert torch.allclose(y, torch.full_like(y, c / math.sqrt(c * c + eps)))
    tiny = torch.full((1, 4), 1e-4, dtype=D)          # mean square 1e-8: eps decides the result
    a = pm.rms_norm(tiny, torch.ones(4, dtype=D), 1e-6)
    b = pm.rms_norm(tiny, torch.ones(4, dtype=D), 1e-5)
    assert torch.allclose(a, tiny / math.sqrt(1e-8 + 1e-6)) and torch.allclose(b, tiny / math.sqrt(1e-8 + 1e-5))
    assert not torch.allclose(a, tiny / (math.sqrt(1e-8) + 1e-6))   # eps outside the root would give this


def test_rms_norm_equals_the_library_and_ignores_scale():
    x, w = rand(5, 24), rand(24)
    assert torch.allclose(pm.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), w, 1e-5))
    assert torch.allclose(pm.rms_norm(1e3 * x, w, 1e-6), pm.rms_norm(1e4 * x, w, 1e-6), atol=1e-7)
    mean_centred = (x - x.mean(-1, keepdim=True)) / x.std(-1, keepdim=True, unbiased=False) * w
    assert not torch.allclose(pm.rms_norm(x, w, 0.0), mean_centred)  # it is not LayerNorm


# ---- linear -------------------------------------------------------------------------------
def test_linear_layout_is_out_by_in():
    x, w, b = rand(3, 7), rand(5, 7), rand(5)
    assert torch.allclose(pm.linear(x, w, b), F.linear(x, w, b))
    assert pm.linear(x, w).shape == (3, 5)


# ---- rotary -------------------------------------------------------------------------------
def test_rope_one_hot_probe_fixes_pairing_sign_and_frequency():
    d, theta = 8, 10000.0
    e0 = torch.zeros(1, 1, d, dtype=D); e0[0, 0, 0] = 1.0
    y = pm.rope_split_half(e0, [1], theta)[0, 0]
    want = torch.zeros(d, dtype=D); want[0] = math.cos(1.0); want[d // 2] = math.sin(1.0)
    assert torch.allclose(y, want)                    # partner of element 0 is d/2, +sin lands there
    e1 = torch.zeros(1, 1, d, dtype=D); e1[0, 0, 1] = 1.0
    a = 3 * theta ** (-2.0 / d)                       # pair 1 at position 3
    y = pm.rope_split_half(e1, [3], theta)[0, 0]
    assert math.isclose(float(y[1]), math.cos(a)) and math.isclose(float(y[1 + d // 2]), math.sin(a))
    eh = torch.zeros(1, 1, d, dtype=D); eh[0, 0, d // 2] = 1.0
    y = pm.rope_split_half(eh, [1], theta)[0, 0]
    assert math.isclose(float(y[0]), -math.sin(1.0)) and math.isclose(float(y[d // 2]), math.cos(1.0))
    y = pm.rope_consecutive(e0, [1], theta)[0, 0]     # the other pairing sends it to element 1
    assert math.isclose(float(y[0]), math.cos(1.0)) and math.isclose(float(y[1]), math.sin(1.0))


def test_rope_identity_norms_and_relative_positions():
    d, theta = 24, 1e6
    q, k = rand(1, 2, d), rand(1, 2, d)
    assert torch.allclose(pm.rope_split_half(q, [0], theta), q)
    r = pm.rope_split_half(q, [17], theta)
    pair = lambda t: t[..., : d // 2] ** 2 + t[..., d // 2:] ** 2
    assert torch.allclose(pair(r), pair(q))
    dot = lambda m, n: (pm.rope_split_half(q, [m], theta) * pm.rope_split_half(k, [n], theta)).sum(-1)
    assert torch.allclose(dot(5, 2), dot(105, 102)) and torch.allclose(dot(9, 9), (q * k).sum(-1))
    assert not torch.allclose(dot(5, 2), dot(2, 5))


# ---- attention ------------------------------------------------------------------------------
def test_rope_angles_formed_in_32_bits():
    """The option for long sequences: the angle is the float32 product of the position and the float32 frequency.  At
    small positions that is the exact angle to 1e-6; at position 30,000 it is tens of microradians to a milliradian off on the fast pairs,
    exactly as numpy's float32 product says."""
    import numpy as np
    d, theta = 16, 1000000.0
    x = torch.zeros(2, 1, d, dtype=D)
    x[:, 0, 0] = 1.0                                     # (1, 0) on pair 0, whose frequency is 1
    x[:, 0, 1] = 1.0                                     # and on pair 1: theta^(-2/16)
    exact = pm.rope_split_half(x, [7, 30001], theta)
    got = pm.rope_split_half(x, [7, 30001], theta, angle_dtype=torch.float32)
    assert torch.allclose(got[0], exact[0], atol=1e-6)
    f1 = np.float32(1.0 / theta ** (2.0 / d))
    a = float(np.float32(30001) * f1)                    # the 32-bit product
    assert abs(a - 30001 / theta ** (2.0 / d)) > 2e-5   # ... is not the exact angle
    assert abs(float(got[1, 0, 1]) - math.cos(a)) < 1e-12 and abs(float(got[1, 0, 1 + d // 2]) - math.sin(a)) < 1e-12
    assert abs(float(got[1, 0, 0]) - math.cos(30001.0)) < 1e-12          # pair 0: position times 1 is exact in 32 bits


def test_attention_special_cases():
    d = 16
    q, k, v = rand(1, 4, d), rand(1, 2, d), rand(1, 2, d)
    o = pm.attention(q, k, v)                          # one key: the output is its value
    assert torch.allclose(o[0, 0], v[0, 0]) and torch.allclose(o[0, 3], v[0, 1])
    S = 6
    q, v = torch.zeros(S, 1, d, dtype=D), rand(S, 1, d)
    o = pm.attention(q, rand(S, 1, d), v)              # equal scores: the mean of the visible values
    for i in range(S):
        assert torch.allclose(o[i, 0], v[: i + 1, 0].mean(0))


def test_attention_equals_the_library_with_repeated_kv_heads():
    S, nH, nKV, d = 9, 6, 2, 24
    q, k, v = rand(S, nH, d), rand(S, nKV, d), rand(S, nKV, d)
    rep = lambda t: t.repeat_interleave(nH // nKV, dim=1).transpose(0, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), rep(k), rep(v), is_causal=True).transpose(0, 1)
    assert torch.allclose(pm.attention(q, k, v), want)
    one = pm.attention(q[:, :1], k[:, :1], v[:, :1])   # one head, last row sees everything: plain softmax
    s = torch.softmax(q[-1, 0] @ k[:, 0].t() / math.sqrt(d), -1)
    assert torch.allclose(one[-1, 0], s @ v[:, 0])
    wrong_map = pm.attention(q, k.flip(1), v.flip(1))   # head 0 must read kv head 0, not the last one
    assert not torch.allclose(wrong_map, want)


def test_attention_causality_past_and_window():
    S, d = 12, 16
    q, k, v = rand(S, 2, d), rand(S, 1, d), rand(S, 1, d)
    full = pm.attention(q, k, v)
    k2, v2 = k.clone(), v.clone(); k2[-1] += 1.0; v2[-1] -= 2.0
    assert torch.allclose(pm.attention(q, k2, v2)[:-1], full[:-1])       # the future never leaks back
    assert torch.allclose(pm.attention(q[-5:], k, v), full[-5:])         # a chunk with a past (limit kv_len-S+i)
    assert torch.allclose(pm.attention(q, k, v, window=S), full)
    assert torch.allclose(pm.attention(q, k, v, window=1), v.expand(S, 2, d))
    w3 = pm.attention(q, k, v, window=3)
    assert torch.allclose(w3[7], pm.attention(q[7:8], k[5:8], v[5:8])[0])  # positions 5, 6, 7 only
    assert torch.allclose(w3[1], full[1]) and not torch.allclose(w3[7], full[7])


def test_attention_scale_is_one_over_sqrt_d():
    S, d = 5, 16
    q, k, v = rand(S, 1, d), rand(S, 1, d), rand(S, 1, d)
    assert torch.allclose(pm.attention(q, k, v), pm.attention(q, k, v, scale=1 / math.sqrt(d)))
    assert not torch.allclose(pm.attention(q, k, v), pm.attention(q, k, v, scale=1 / d))


# ---- SwiGLU ---------------------------------------------------------------------------------
def test_swiglu():
    x = rand(4, 10); wg, wu, wd = rand(14, 10), rand(14, 10), rand(10, 14)
    assert torch.allclose(pm.swiglu(x, wg, wu, wd), F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd))
    eye = torch.eye(3, dtype=D)
    g = torch.tensor([[0.0, 30.0, -30.0]], dtype=D)
    ones = torch.ones(3, 3, dtype=D) / 3
    y = pm.swiglu(g, eye, eye, eye)                     # silu(g) * g
    assert torch.allclose(y, torch.tensor([[0.0, 900.0, 0.0]], dtype=D), atol=1e-9)
    assert not torch.allclose(pm.swiglu(x, wg, wu, wd), pm.swiglu(x, wu, wg, wd))  # gate and up are not symmetric


# ---- whole model ----------------------------------------------------------------------------
def random_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    H, V, I = cfg["hidden_size"], cfg["vocab_size"], cfg["intermediate_size"]
    nH, nKV, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    r = lambda *s: (torch.randn(*s, generator=g, dtype=D) * 0.05)
    W = {"model.embed_tokens.weight": r(V, H), "model.norm.weight": 1 + r(H)}
    if not cfg["tie_word_embeddings"]:
        W["lm_head.weight"] = r(V, H)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}"
        W.update({f"{p}.input_layernorm.weight": 1 + r(H), f"{p}.post_attention_layernorm.weight": 1 + r(H),
                  f"{p}.self_attn.q_proj.weight": r(nH * d, H), f"{p}.self_attn.k_proj.weight": r(nKV * d, H),
                  f"{p}.self_attn.v_proj.weight": r(nKV * d, H), f"{p}.self_attn.o_proj.weight": r(H, nH * d),
                  f"{p}.mlp.gate_proj.weight": r(I, H), f"{p}.mlp.up_proj.weight": r(I, H),
                  f"{p}.mlp.down_proj.weight": r(H, I)})
        if cfg["attention_bias"]:
            W.update({f"{p}.self_attn.q_proj.bias": r(nH * d), f"{p}.self_attn.k_proj.bias": r(nKV * d),
                      f"{p}.self_attn.v_proj.bias": r(nKV * d)})
    return W


@pytest.mark.parametrize("name", list(TINY))
def test_residual_structure_and_head(name):
    cfg = TINY[name]
    W = random_weights(cfg)
    ids = [3, 7, 1, 7, 250, 9]
    Z = dict(W)
    for l in range(cfg["num_hidden_layers"]):             # silence both sub-blocks: only the stream is left
        Z[f"model.layers.{l}.self_attn.o_proj.weight"] = torch.zeros_like(W[f"model.layers.{l}.self_attn.o_proj.weight"])
        Z[f"model.layers.{l}.mlp.down_proj.weight"] = torch.zeros_like(W[f"model.layers.{l}.mlp.down_proj.weight"])
    head = Z.get("lm_head.weight", Z["model.embed_tokens.weight"])
    want = pm.rms_norm(Z["model.embed_tokens.weight"][ids], Z["model.norm.weight"], cfg["rms_norm_eps"]) @ head.t()
    assert torch.allclose(pm.forward(cfg, Z, ids), want)
    base = pm.forward(cfg, W, ids)
    if cfg["tie_word_embeddings"]:
        assert "lm_head.weight" not in W
    else:
        W2 = dict(W); W2["lm_head.weight"] = W["lm_head.weight"] * 2
        assert torch.allclose(pm.forward(cfg, W2, ids), 2 * base)       # the head alone scales the logits
    ids2 = list(ids); ids2[-1] = 11
    assert torch.allclose(pm.forward(cfg, W, ids2)[:-1], base[:-1])      # causal end to end
    assert not torch.allclose(pm.forward(cfg, W, ids2)[-1], base[-1])


@pytest.mark.parametrize("name", list(TINY))
def test_only_distances_count(name):
    cfg = TINY[name]
    W = random_weights(cfg, 1)
    ids = list(range(40, 70))                             # longer than C's window
    base = pm.forward(cfg, W, ids)
    assert torch.allclose(pm.forward(cfg, W, ids, positions=range(100, 130)), base, atol=1e-9)
    assert not torch.allclose(pm.forward(cfg, W, ids, positions=range(0, 60, 2)), base, atol=1e-6)


@pytest.mark.parametrize("name", list(TINY))
def test_rows_of_a_one_layer_model_equal_the_whole_forward(name):
    """The oracle for long sequences at real widths computes everything but keys and values for the wanted rows alone:
    the same logits as the whole forward, with C's window (on its only layer) and without."""
    cfg = dict(TINY[name], num_hidden_layers=1, max_window_layers=0)
    W = random_weights(cfg, 3)
    ids = [(7 * i + 3) % cfg["vocab_size"] for i in range(50)]
    rows = [0, 1, 23, 24, 25, 48, 49]
    assert torch.allclose(pm.forward_rows_one_layer(cfg, W, ids, rows), pm.forward(cfg, W, ids)[rows], atol=1e-12)
    with pytest.raises(ValueError):
        pm.forward_rows_one_layer(TINY[name], random_weights(TINY[name]), ids, rows)


def test_window_changes_only_windowed_layers_reach():
    cfg = TINY["C"]
    W = random_weights(cfg, 2)
    ids = list(range(30))
    nowin = dict(cfg, use_sliding_window=False)
    a, b = pm.forward(cfg, W, ids), pm.forward(nowin, W, ids)
    assert torch.allclose(a[:24], b[:24]) and not torch.allclose(a[24:], b[24:])   # window 24: first 24 rows see all
    assert [pm.layer_window(cfg, l) for l in range(4)] == [None, 24, 24, 24]


# ---- sampling -------------------------------------------------------------------------------
def test_penalties_formula():
    l = torch.tensor([2.0, -2.0, 1.0, 0.5])
    out = pm.apply_penalties(l, [0, 1, 1], repetition=2.0, frequency=0.25, presence=0.5)
    assert torch.allclose(out, torch.tensor([2.0 / 2 - 0.25 - 0.5, -2.0 * 2 - 0.5 - 0.5, 1.0, 0.5]))


def test_top_p_keeps_the_crossing_token_and_top_k_min_p():
    logits = torch.log(torch.tensor([0.5, 0.3, 0.15, 0.05]))
    p = pm.filtered_probs(logits, 1.0, top_p=0.6)
    assert (p > 0).tolist() == [True, True, False, False]              # 0.5 < 0.6 <= 0.8: the crossing one stays
    assert (pm.filtered_probs(logits, 1.0, top_p=0.5) > 0).tolist() == [True, False, False, False]
    assert (pm.filtered_probs(logits, 1.0, top_k=3) > 0).tolist() == [True, True, True, False]
    assert (pm.filtered_probs(logits, 1.0, min_p=0.5) > 0).tolist() == [True, True, False, False]
    assert (pm.filtered_probs(logits, 1.0, top_k=3, top_p=0.9) > 0).tolist() == [True, True, True, False]
    assert torch.allclose(pm.filtered_probs(logits, 1.0), torch.tensor([0.5, 0.3, 0.15, 0.05], dtype=D))
    sharp = pm.filtered_probs(logits, 0.5)
    assert torch.allclose(sharp, torch.tensor([0.25, 0.09, 0.0225, 0.0025], dtype=D) / 0.365)


def test_cdf_walk():
    w = torch.tensor([0.0, 0.2, 0.0, 0.6, 0.2], dtype=D)
    assert [pm.cdf_walk(w, u) for u in (0.0, 0.19, 0.2, 0.79, 0.8, 0.999)] == [1, 1, 3, 3, 4, 4]
    assert pm.cdf_walk(w, 1.0) == 4                                     # fallback: the last kept index
