"""Slow float64 oracle for the Nanurax design, one function per mechanism.

Written from the design's equations only; it shares no code with the
engine (no ops, no model classes, no cache): sequences are plain
[tokens, width] tensors, the recurrent state is a Python-held matrix per
head, attention sees the whole sequence at once through an explicit mask.

Weights come as a dict name -> tensor using the checkpoint's own names
("l<i>.mix.k", "l<i>.mlp.e<j>.gate", ...); the configuration is the parsed
config.json dict.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.to(F64)


def unit_rms(x, eps):
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(
        math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def lin(w, h):
    return h.to(F64) @ w.to(F64).T


def dense_ff(h, gate, up, down):
    return lin(down, gelu_tanh(lin(gate, h)) * lin(up, h))


def expert_ff(h, gate, up, down, limit):
    g = torch.clamp(lin(gate, h), max=limit)
    u = torch.clamp(lin(up, h), min=-limit, max=limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return lin(down, y)


def moe_ff(h, W, pre, spec):
    """h [T, width]; returns [T, width]."""
    n_exp = spec["router"]["experts"]
    top = spec["router"]["top"]
    limit = spec["expert"]["limit"]
    s = torch.sigmoid(lin(W[pre + "router"], h))      # [T, E]
    out = torch.zeros_like(h, dtype=F64)
    for t in range(h.shape[0]):
        order = sorted(range(n_exp), key=lambda e: -float(s[t, e]))[:top]
        for e in order:
            ep = f"{pre}e{e}."
            out[t] += expert_ff(
                (s[t, e] * h[t].to(F64))[None], W[ep + "gate"],
                W[ep + "up"], W[ep + "down"], limit)[0]
    if spec.get("shared"):
        sp = pre + "shared."
        sh = expert_ff(h, W[sp + "gate"], W[sp + "up"], W[sp + "down"],
                       spec["shared"]["limit"])
        out = out + sh * torch.sigmoid(lin(W[sp + "sg"], h))
    return out


def general_delta(h, W, pre, spec, eps, state=None):
    """h [T, width]. state: [heads, dim, dim] float64 or None (zeros).
    Returns (out [T, width], new state)."""
    H, D = spec["heads"], spec["dim"]
    T = h.shape[0]
    r = lin(W[pre + "r"], h).view(T, H, D)
    k = lin(W[pre + "k"], h).view(T, H, D)
    v = lin(W[pre + "v"], h).view(T, H, D)
    zw = lin(W[pre + "w2"], torch.tanh(lin(W[pre + "w1"], h))) \
        + W[pre + "w0"].to(F64)
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(zw)).view(T, H, D)
    a = torch.sigmoid(lin(W[pre + "a"], h)
                      + W[pre + "a.b"].to(F64)).view(T, H, D)
    S = torch.zeros(H, D, D, dtype=F64) if state is None else state.clone()
    o = torch.zeros(T, H, D, dtype=F64)
    for t in range(T):
        for hd in range(H):
            kk = k[t, hd]
            u = kk / torch.sqrt((kk * kk).sum() + 1e-6)
            old = S[hd]
            S[hd] = (w[t, hd][:, None] * old
                     - torch.outer(a[t, hd] * u, u @ old)
                     + torch.outer(kk, v[t, hd]))
            o[t, hd] = S[hd].T @ r[t, hd]
    o = unit_rms(o, eps).reshape(T, H * D) * W[pre + "norm"].to(F64)
    o = o * torch.sigmoid(lin(W[pre + "g"], h))
    return lin(W[pre + "o"], o), S


def attention(h, W, pre, spec, positions=None):
    """Whole-sequence attention; h [T, width], positions default 0..T-1."""
    H, G = spec["heads"], spec.get("kv_heads", spec["heads"])
    D, DV = spec["dim"], spec.get("vdim", spec["dim"])
    size = spec["mask"]["size"]
    T = h.shape[0]
    pos = torch.arange(T) if positions is None else positions
    q = lin(W[pre + "q"], h).view(T, H, D)
    k = lin(W[pre + "k"], h).view(T, G, D)
    v = lin(W[pre + "v"], h).view(T, G, DV)
    rep = H // G
    score = torch.zeros(H, T, T, dtype=F64)
    for hd in range(H):
        score[hd] = (q[:, hd] @ k[:, hd // rep].T) * spec["scale"]
    score = torch.einsum("hg,gij->hij", W[pre + "talk"].to(F64), score)
    see = (pos[None, :] <= pos[:, None]) & (
        (pos[None, :] // size) == (pos[:, None] // size))
    out = torch.zeros(T, H, DV, dtype=F64)
    for hd in range(H):
        e = torch.where(see, torch.exp(score[hd]),
                        torch.zeros((), dtype=F64))
        p = e / (1.0 + e.sum(-1, keepdim=True))
        out[:, hd] = p @ v[:, hd // rep]
    return lin(W[pre + "o"], out.reshape(T, H * DV))


def forward(cfg, W, tokens, return_layers=False):
    """Full-prompt forward: logits [T, vocab] float64 (and the residual
    stream after every layer when asked)."""
    eps = cfg["norm"]["eps"]
    x = W["embed"].to(F64)[torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = rms_norm(x, W[pre + "norm1"], eps)
        if layer["type"] == "general_delta":
            m, _ = general_delta(h, W, pre + "mix.", layer["mixer"], eps)
        elif layer["type"] == "attention":
            m = attention(h, W, pre + "mix.", layer["mixer"])
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is None:
            f = 0.0
        elif mlp["kind"] == "dense":
            f = dense_ff(h, W[pre + "mlp.gate"], W[pre + "mlp.up"],
                         W[pre + "mlp.down"])
        else:
            f = moe_ff(h, W, pre + "mlp.", mlp)
        x = x + (m + f)
        streams.append(x.clone())
    logits = lin(W["head"], rms_norm(x, W["final.norm"], eps))
    if return_layers:
        return logits, torch.stack(streams)
    return logits
