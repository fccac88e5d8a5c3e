"""Slow float64 oracle for the Derusun design, one function per mechanism.

Written from the design's equations only; it shares no code with the engine
(no ops, no model classes, no cache, no state slots): a sequence is a plain
[tokens, width] tensor processed whole, the recurrence is a Python loop over
tokens, attention sees every key at once through an explicit visibility
mask.

Weights come as a dict name -> tensor under the checkpoint's own names
("l<i>.mix.q", "l<i>.mlp.gate", ...); the configuration is the parsed
config.json dict.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def lin(w, h, b=None):
    y = h.to(F64) @ w.to(F64).T
    return y if b is None else y + b.to(F64)


def group_rms_norm(x, w, eps, groups=1):
    """Each of `groups` equal consecutive parts of the last axis is divided
    by its own root mean square; the whole is scaled by w."""
    x = x.to(F64)
    sh = x.shape
    p = x.reshape(*sh[:-1], groups, sh[-1] // groups)
    p = p / torch.sqrt((p * p).mean(-1, keepdim=True) + eps)
    return p.reshape(sh) * w.to(F64)


def token_shift(h, mu, prev=None):
    """h_t <- h_t + (h_{t-1} - h_t) * mu with the un-shifted predecessor;
    the token before the first one is `prev` (zeros when None)."""
    h = h.to(F64)
    first = torch.zeros_like(h[:1]) if prev is None else prev.to(F64)[None]
    before = torch.cat([first, h[:-1]], dim=0)
    return h + (before - h) * mu.to(F64)


def depth_average(history, weights):
    """sum_j weights[j] * history[j] over the streams seen so far."""
    out = torch.zeros_like(history[0], dtype=F64)
    for j, xj in enumerate(history):
        out = out + weights[j].to(F64) * xj.to(F64)
    return out


def clamped_ff(h, gate, up, down, limit):
    g = torch.clamp(lin(gate, h), max=limit)
    u = torch.clamp(lin(up, h), min=-limit, max=limit)
    return lin(down, g * torch.sigmoid(1.702 * g) * (u + 1.0))


def causal_conv_silu(x, taps_w):
    """x [T, C]; taps_w [C, K], last column weighs the current token;
    nothing before the first token."""
    x = x.to(F64)
    T, C = x.shape
    K = taps_w.shape[1]
    w = taps_w.to(F64)
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(K):
            s = t - (K - 1) + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y * torch.sigmoid(y)


def channel_delta(h, W, pre, m, eps):
    """Gated delta rule with one decay per head and key channel."""
    H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    rep = H // G
    q = causal_conv_silu(lin(W[pre + "q"], h), W[pre + "q.conv"])
    k = causal_conv_silu(lin(W[pre + "k"], h), W[pre + "k.conv"])
    v = causal_conv_silu(lin(W[pre + "v"], h), W[pre + "v.conv"])
    q = q.view(T, G, D)
    k = k.view(T, G, D)
    v = v.view(T, H, DV)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(lin(W[pre + "b"], h))                   # [T, H]
    z = lin(W[pre + "a2"], lin(W[pre + "a1"], h)) + W[pre + "dt_bias"].to(F64)
    rate = torch.exp(W[pre + "A_log"].to(F64))                   # [H]
    decay = torch.exp(-rate[None, :, None]
                      * torch.nn.functional.softplus(z).view(T, H, D))
    gate = torch.sigmoid(lin(W[pre + "g2"], lin(W[pre + "g1"], h)))
    gate = gate.view(T, H, DV)
    out = torch.zeros(T, H, DV, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, DV, dtype=F64)
        for t in range(T):
            kk, qq = k[t, hd // rep], q[t, hd // rep]
            S = decay[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ kk)
            S = S + kk[:, None] * u[None, :]
            out[t, hd] = S.T @ qq
    out = out / torch.sqrt((out * out).mean(-1, keepdim=True) + eps)
    out = out * W[pre + "norm"].to(F64) * gate
    return lin(W[pre + "o"], out.reshape(T, H * DV))


def sink_softmax(scores, visible, sink):
    """scores [H, T, T], visible [T, T] bool, sink [H]: softmax over the
    visible keys whose denominator also holds exp(sink_h)."""
    s = scores.masked_fill(~visible[None], -math.inf)
    m = torch.maximum(s.max(-1, keepdim=True).values,
                      sink.to(F64)[:, None, None])
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True)
                + torch.exp(sink.to(F64)[:, None, None] - m))


def window_visibility(T, size, keep_first):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def attention(h, W, pre, m, eps, v_first=None):
    """Windowed grouped-query attention with biases, per-head query/key
    norm, capped scores, kept first keys and a learned sink. Returns
    (out, this layer's cached values [T, G, DV])."""
    H, G, D, DV = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    rep = H // G
    q = lin(W[pre + "q"], h, W[pre + "q.b"]).view(T, H, D)
    k = lin(W[pre + "k"], h, W[pre + "k.b"]).view(T, G, D)
    v = lin(W[pre + "v"], h, W[pre + "v.b"]).view(T, G, DV)
    q = group_rms_norm(q, W[pre + "q.norm"], eps)
    k = group_rms_norm(k, W[pre + "k.norm"], eps)
    if m.get("v_mix") and v_first is not None:
        lam = W[pre + "vmix"].to(F64)
        v = (1.0 - lam) * v + lam * v_first.to(F64)
    kk = k.repeat_interleave(rep, dim=1)
    vv = v.repeat_interleave(rep, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * m["scale"]
    cap = m.get("softcap")
    if cap:
        s = cap * torch.tanh(s / cap)
    mask = m.get("mask") or {}
    vis = window_visibility(T, mask.get("size", T), mask.get("keep_first", 0))
    p = sink_softmax(s, vis, W[pre + "sink"])
    o = torch.einsum("hij,jhv->ihv", p, vv).reshape(T, H * DV)
    return lin(W[pre + "o"], o), v


def rotate_pairs(x, positions, base, dims):
    """Pairs (2i, 2i+1) of the first `dims` entries of the last axis turn
    by the angle position * base^(-2i/dims)."""
    x = x.to(F64).clone()
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)],
                     dtype=F64)
    a = positions.to(F64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
    u, w = x[..., 0:dims:2].clone(), x[..., 1:dims:2].clone()
    x[..., 0:dims:2] = u * c - w * s
    x[..., 1:dims:2] = w * c + u * s
    return x


def latent_attention(h, W, pre, m, eps, positions=None):
    """Keys and values of all heads are expanded from one low-rank latent
    per token; one rotated key part is shared by the heads."""
    H, D, R, DV, L = (m["heads"], m["dim"], m["rot_dim"], m["vdim"],
                      m["kv_rank"])
    T = h.shape[0]
    if positions is None:
        positions = torch.arange(T)
    rot = m["rot"]
    q = lin(W[pre + "q"], h).view(T, H, D + R)
    qa, qr = q[..., :D], q[..., D:]
    dkv = lin(W[pre + "dkv"], h)
    c = group_rms_norm(dkv[:, :L], W[pre + "dkv.norm"], eps)
    kr = rotate_pairs(dkv[:, L:], positions, rot["base"], rot["dims"])
    qr = rotate_pairs(qr, positions, rot["base"], rot["dims"])
    ka = lin(W[pre + "uk"], c).view(T, H, D)
    vv = lin(W[pre + "uv"], c).view(T, H, DV)
    s = (torch.einsum("ihd,jhd->hij", qa, ka)
         + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    vis = window_visibility(T, T, 0)
    p = sink_softmax(s, vis, W[pre + "sink"])
    o = torch.einsum("hij,jhv->ihv", p, vv).reshape(T, H * DV)
    return lin(W[pre + "o"], o)


def forward(cfg, W, tokens, layer_outputs=None):
    """tokens: list[int] -> logits [T, vocab] float64. layer_outputs: an
    optional list that receives the residual stream after every layer."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    x = W["embed"].to(F64)[torch.tensor(tokens)]
    history = [x]
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        m = layer["mixer"]
        h = group_rms_norm(x, W[pre + "norm1"], eps, groups)
        h = token_shift(h, W[pre + "shift"])
        kind = layer["type"]
        if kind == "channel_delta":
            y = channel_delta(h, W, pre + "mix.", m, eps)
        elif kind == "attention":
            y, v = attention(h, W, pre + "mix.", m, eps, v_first)
            if m.get("v_mix") and v_first is None:
                v_first = v
        elif kind == "latent_attention":
            y = latent_attention(h, W, pre + "mix.", m, eps)
        else:
            raise ValueError(kind)
        x = x + y
        ml = layer.get("mlp")
        if ml is not None:
            h2 = group_rms_norm(x, W[pre + "norm2"], eps, groups)
            x = x + clamped_ff(h2, W[pre + "mlp.gate"], W[pre + "mlp.up"],
                               W[pre + "mlp.down"], ml["limit"])
        history.append(x)
        x = depth_average(history, W[pre + "dwa"])
        if layer_outputs is not None:
            layer_outputs.append(x)
    h = group_rms_norm(x, W["final.norm"], eps, groups)
    return lin(W["head"], h)
