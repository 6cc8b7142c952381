"""A plain, slow implementation of the Qwen2.5 dense decoder, written from the reference's formulas.

Whole sequences, no cache, one function per part, on the CPU.  It shares no code with the
engine: it reads config.json with json and model.safetensors with the safetensors package,
and takes every size from the config dict.  Each function cites the reference lines
(paths relative to the reference's root) that fix its formula.

``dtype`` is the arithmetic type (float32 as the reference computes, or float64 for a tighter
oracle).
"""
import json
import math
import os

import torch


def load_folder(folder, dtype=torch.float32):
    """config.json as a dict and all tensors widened to ``dtype``."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {k: v.to(dtype) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, tensors


def embedding(ids, table):
    """x[t, :] = E[id[t], :], no scaling.
    runtime/backends/cuda/native/cuda_kernels.cu:255-270"""
    return table[torch.as_tensor(ids, dtype=torch.long)]


def rms_norm(x, w, eps):
    """y_i = x_i * rsqrt(mean(x^2) + eps) * w_i, eps inside the square root.
    runtime/backends/cuda/native/cuda_kernels.cu:15-48 (line 41)"""
    ms = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * torch.rsqrt(ms + eps) * w


def linear(x, w, b=None):
    """y = x W^T (+ b) with W stored [out, in].
    runtime/backends/cuda/native/cublas_gemm.cpp:99-117; bias cuda_kernels.cu:518-527"""
    y = x @ w.t()
    return y if b is None else y + b


def rope_split_half(x, positions, theta, angle_dtype=None):
    """x [S, heads, d]; pair p joins elements p and p + d/2; f_p = 1 / theta^(2p/d);
    (x0, x1) <- (x0 cos a - x1 sin a, x0 sin a + x1 cos a) with a = position * f_p.
    runtime/backends/cuda/native/cuda_kernels.cu:71-117 (pairing 102-105); the same oracle as
    tests/unit/test_native_forward.cpp:71-106 with rope_type 2.

    ``angle_dtype`` torch.float32: the angle is the 32-bit product of the position and the frequency rounded to 32
    bits, as the reference forms it (float freq, float angle: cuda_kernels.cu:91-96); its cosine and sine are then
    taken in x's type.  At positions beyond ten thousand that rounding (up to 1e-3 rad on the fast pairs) is part of
    the function a 32-bit implementation computes; without it (the default) the angle is exact in x's type."""
    S, h, d = x.shape
    half = d // 2
    p = torch.arange(half, dtype=x.dtype)
    freq = 1.0 / torch.pow(torch.tensor(theta, dtype=x.dtype), 2.0 * p / d)
    if angle_dtype is not None:
        ang = (torch.as_tensor(positions).to(angle_dtype)[:, None] * freq.to(angle_dtype)[None, :]).to(x.dtype)
    else:
        ang = torch.as_tensor(positions, dtype=x.dtype)[:, None] * freq[None, :]  # [S, half]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    x0, x1 = x[..., :half], x[..., half:]
    return torch.cat([x0 * cos - x1 * sin, x0 * sin + x1 * cos], dim=-1)


def rope_consecutive(x, positions, theta):
    """The other pairing the reference knows (rope_type 0): pairs (2p, 2p+1).
    runtime/backends/cuda/native/cuda_kernels.cu:106-110.  Not used by qwen2; kept to pin the
    kernel's second style."""
    S, h, d = x.shape
    half = d // 2
    p = torch.arange(half, dtype=x.dtype)
    freq = 1.0 / torch.pow(torch.tensor(theta, dtype=x.dtype), 2.0 * p / d)
    ang = torch.as_tensor(positions, dtype=x.dtype)[:, None] * freq[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    x0, x1 = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = x0 * cos - x1 * sin
    out[..., 1::2] = x0 * sin + x1 * cos
    return out


def attention(q, k, v, scale=None, window=None, q_positions=None, k_positions=None):
    """Causal grouped-query attention, every key visible up to the query's own position.

    q [Sq, nH, d], k and v [Sk, nKV, d].  Head h reads kv head h // (nH // nKV)
    (runtime/backends/cuda/kernels/flash_attention.cu:71-72); query at position p sees keys at
    positions j <= p (flash_attention.cu:86) and, with a window W, j > p - W (no counterpart in
    the reference, which has no window); s = (q . k) * scale with scale = 1/sqrt(d) applied
    after the dot product (flash_attention.cu:144; transformer_forward.cu:2125-2130);
    o = softmax(s) v (flash_attention.cu:152-173), 0 where no key is visible.
    Positions default to 0..S-1 with the queries at the end of the keys (a chunk with a past:
    limit kv_len - S + i, as in tests/unit/test_fa2_prefill.cu:98).
    """
    Sq, nH, d = q.shape
    Sk, nKV, _ = k.shape
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    kp = torch.arange(Sk) if k_positions is None else torch.as_tensor(k_positions)
    qp = torch.arange(Sk - Sq, Sk) if q_positions is None else torch.as_tensor(q_positions)
    visible = kp[None, :] <= qp[:, None]
    if window is not None:
        visible &= kp[None, :] > qp[:, None] - window
    out = torch.zeros_like(q)
    ratio = nH // nKV
    for h in range(nH):
        g = h // ratio
        s = (q[:, h, :] @ k[:, g, :].t()) * scale
        s = s.masked_fill(~visible, float("-inf"))
        m = s.max(dim=-1, keepdim=True).values
        m = torch.where(torch.isfinite(m), m, torch.zeros_like(m))
        e = torch.exp(s - m)
        l = e.sum(dim=-1, keepdim=True)
        pr = torch.where(l > 0, e / torch.where(l > 0, l, torch.ones_like(l)), torch.zeros_like(e))
        out[:, h, :] = pr @ v[:, g, :]
    return out


def swiglu(x, w_gate, w_up, w_down):
    """a = g / (1 + exp(-g)) * u with g = x Wg^T, u = x Wu^T; y = a Wd^T; no biases.
    runtime/backends/cuda/native/cuda_kernels.cu:139-151;
    runtime/backends/cuda/native/transformer_forward.cu:2383-2419, 2487-2494, 2528-2547"""
    g, u = linear(x, w_gate), linear(x, w_up)
    return linear(g / (1.0 + torch.exp(-g)) * u, w_down)


def layer_window(cfg, layer):
    """Layers at or beyond max_window_layers use the window when use_sliding_window is set.
    The reference reads none of these keys; the engine fixes this meaning itself."""
    if cfg.get("use_sliding_window") and layer >= cfg.get("max_window_layers", 0):
        return cfg["sliding_window"]
    return None


def attention_block(x, W, cfg, layer, positions):
    """q/k/v projections with optional bias, rotary on q and k, attention, output projection.
    runtime/backends/cuda/native/transformer_forward.cu:1944-2135 (bias presence by tensor
    presence: runtime/backends/cuda/native/weight_map.cpp:55-58), 2145-2241."""
    p = f"model.layers.{layer}.self_attn"
    nH, nKV = cfg["num_attention_heads"], cfg.get("num_key_value_heads", cfg["num_attention_heads"])
    d = cfg.get("head_dim") or cfg["hidden_size"] // nH
    S = x.shape[0]
    q = linear(x, W[f"{p}.q_proj.weight"], W.get(f"{p}.q_proj.bias")).view(S, nH, d)
    k = linear(x, W[f"{p}.k_proj.weight"], W.get(f"{p}.k_proj.bias")).view(S, nKV, d)
    v = linear(x, W[f"{p}.v_proj.weight"], W.get(f"{p}.v_proj.bias")).view(S, nKV, d)
    theta = cfg.get("rope_theta", 10000.0)
    q, k = rope_split_half(q, positions, theta), rope_split_half(k, positions, theta)
    o = attention(q, k, v, window=layer_window(cfg, layer), q_positions=positions, k_positions=positions)
    return linear(o.reshape(S, nH * d), W[f"{p}.o_proj.weight"])


def forward(cfg, W, ids, positions=None):
    """Logits [S, V] of a whole sequence.  Pre-norm blocks, residual adds, final norm, head
    (tied to the embedding when the file has no lm_head.weight).
    runtime/backends/cuda/native/transformer_forward.cu:1676-2712; tie: weight_map.cpp:33-37"""
    S = len(ids)
    positions = list(range(S)) if positions is None else list(positions)
    eps = cfg.get("rms_norm_eps", 1e-6)
    x = embedding(ids, W["model.embed_tokens.weight"])
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}"
        x = x + attention_block(rms_norm(x, W[f"{p}.input_layernorm.weight"], eps), W, cfg, l, positions)
        h = rms_norm(x, W[f"{p}.post_attention_layernorm.weight"], eps)
        x = x + swiglu(h, W[f"{p}.mlp.gate_proj.weight"], W[f"{p}.mlp.up_proj.weight"], W[f"{p}.mlp.down_proj.weight"])
    h = rms_norm(x, W["model.norm.weight"], eps)
    head = W["lm_head.weight"] if "lm_head.weight" in W else W["model.embed_tokens.weight"]
    return linear(h, head)


def forward_rows_one_layer(cfg, W, ids, rows, angle_dtype=None):
    """Logits [len(rows), V] at the places ``rows`` of a whole sequence, for a model of ONE layer: keys and values need
    the first norm and two projections of every token, everything else is computed for the wanted rows alone, which
    makes sequences of tens of thousands of tokens at real layer widths affordable on the CPU.  The same functions in
    the same order as ``forward`` (a test compares the two).  ``angle_dtype``: see ``rope_split_half``."""
    if cfg["num_hidden_layers"] != 1:
        raise ValueError("forward_rows_one_layer: the second layer's keys would need every row of the first")
    S, rows = len(ids), list(rows)
    positions = list(range(S))
    eps = cfg.get("rms_norm_eps", 1e-6)
    nH, nKV = cfg["num_attention_heads"], cfg.get("num_key_value_heads", cfg["num_attention_heads"])
    d = cfg.get("head_dim") or cfg["hidden_size"] // nH
    theta = cfg.get("rope_theta", 10000.0)
    p, a = "model.layers.0", "model.layers.0.self_attn"
    x = embedding(ids, W["model.embed_tokens.weight"])
    h = rms_norm(x, W[f"{p}.input_layernorm.weight"], eps)
    k = rope_split_half(linear(h, W[f"{a}.k_proj.weight"], W.get(f"{a}.k_proj.bias")).view(S, nKV, d), positions, theta, angle_dtype)
    v = linear(h, W[f"{a}.v_proj.weight"], W.get(f"{a}.v_proj.bias")).view(S, nKV, d)
    q = rope_split_half(linear(h[rows], W[f"{a}.q_proj.weight"], W.get(f"{a}.q_proj.bias")).view(len(rows), nH, d), rows, theta,
                        angle_dtype)
    o = attention(q, k, v, window=layer_window(cfg, 0), q_positions=rows, k_positions=positions)
    xr = x[rows] + linear(o.reshape(len(rows), nH * d), W[f"{a}.o_proj.weight"])
    hr = rms_norm(xr, W[f"{p}.post_attention_layernorm.weight"], eps)
    xr = xr + swiglu(hr, W[f"{p}.mlp.gate_proj.weight"], W[f"{p}.mlp.up_proj.weight"], W[f"{p}.mlp.down_proj.weight"])
    head = W["lm_head.weight"] if "lm_head.weight" in W else W["model.embed_tokens.weight"]
    return linear(rms_norm(xr, W["model.norm.weight"], eps), head)


def greedy_generate(cfg, W, prompt, n_new):
    """Token ids chosen by argmax (lowest index on ties), recomputing the whole sequence."""
    ids = list(prompt)
    for _ in range(n_new):
        logits = forward(cfg, W, ids)[-1]
        ids.append(int(torch.argmax(logits)))
    return ids[len(prompt):]


# ---- sampling ---------------------------------------------------------------------------
def apply_penalties(logits, recent_ids, repetition, frequency, presence):
    """For each distinct recent id with count c: l = l/rep if l > 0 else l*rep; l -= freq*c;
    if c > 0: l -= presence.  runtime/backends/cuda/native/gpu_sampler.cu:22-48"""
    out = logits.clone()
    counts = {}
    for t in recent_ids:
        counts[t] = counts.get(t, 0) + 1
    for t, c in counts.items():
        l = out[t]
        l = l / repetition if l > 0 else l * repetition
        l = l - frequency * c
        if c > 0:
            l = l - presence
        out[t] = l
    return out


def filtered_probs(logits, temperature, top_k=0, top_p=1.0, min_p=0.0):
    """softmax(logits / T) (gpu_sampler.cu:216-267), then top-k (keep the k most probable), then
    top-p over the survivors: in descending probability keep tokens until the running sum reaches
    top_p of the survivors' mass, the crossing token included (gpu_sampler.cu:273-330), then min-p
    (keep p >= min_p * max p).  Unnormalised survivors' probabilities are returned."""
    p = torch.softmax(logits.double() / temperature, dim=-1)
    keep = torch.ones_like(p, dtype=torch.bool)
    order = torch.argsort(p, descending=True, stable=True)
    if 0 < top_k < p.numel():
        keep[order[top_k:]] = False
    if 0.0 < top_p < 1.0:
        ps = p[order] * keep[order]
        need = top_p * ps.sum()
        cum = torch.cumsum(ps, 0)
        n_keep = int((cum < need).sum()) + 1
        keep[order[n_keep:]] = False
    if min_p > 0.0:
        keep &= p >= min_p * p.max()
    return p * keep


def cdf_walk(weights, u):
    """Walk the cumulative sum in index order until u * total < cum; last index as fallback.
    runtime/backends/cuda/native/gpu_sampler.cu:374-401"""
    total = weights.sum()
    cum = torch.cumsum(weights, 0)
    hit = torch.nonzero(u * total < cum)
    return int(hit[0]) if hit.numel() else int(torch.nonzero(weights > 0)[-1])
