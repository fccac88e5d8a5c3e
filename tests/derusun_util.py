"""Helpers for the Derusun tests: small configurations in the checkpoint's
own config.json layout and random bf16 weights under the checkpoint's tensor
names. Checkpoint folders, engines and error measures come from
nanurax_util."""

from __future__ import annotations

import torch

from nanurax_util import (TOL, close, make_engine, rel_err,  # noqa: F401
                          row_errs, save_checkpoint)


def cdelta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3):
    return {"type": "channel_delta",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                      "vdim": vdim, "conv": conv}}


def wattn(heads=6, kv_heads=2, dim=16, vdim=24, size=20, keep=3, scale=0.3,
          cap=8.0, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": scale, "v_mix": v_mix}
    if size:
        m["mask"] = {"size": size, "keep_first": keep}
    if cap:
        m["softcap"] = cap
    return {"type": "attention", "mixer": m}


def lattn(heads=3, dim=16, rot_dim=8, vdim=12, rank=24, scale=0.2,
          base=10000.0, dims=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim,
                      "vdim": vdim, "kv_rank": rank, "scale": scale,
                      "rot": {"base": base,
                              "dims": rot_dim if dims is None else dims}}}


def dense(ff=72, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def make_cfg(layers, width=64, vocab=97, eps=1e-5, groups=2):
    """layers: [(mixer dict, mlp dict | None)]."""
    return {
        "architecture": "Derusun", "vocab": vocab, "width": width,
        "norm": {"eps": eps, "groups": groups},
        "layers": [dict(m, mlp=f) for m, f in layers],
    }


def make_weights(cfg, seed=0, ranks=(6, 5)):
    """ranks: rows of the low-rank decay and output-gate projections."""
    g = torch.Generator().manual_seed(seed)
    W = {}

    def lin(name, out, inp, gain=1.0):
        W[name] = (torch.randn(out, inp, generator=g) * gain
                   / inp ** 0.5).to(torch.bfloat16)

    def vec(name, n, mean=0.0, std=1.0):
        W[name] = (mean + std * torch.randn(n, generator=g)).to(
            torch.bfloat16)

    width, vocab = cfg["width"], cfg["vocab"]
    W["embed"] = torch.randn(vocab, width, generator=g).to(torch.bfloat16)
    lin("head", vocab, width)
    vec("final.norm", width, 1.0, 0.1)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        vec(p + "norm1", width, 1.0, 0.1)
        W[p + "shift"] = torch.rand(width, generator=g).to(torch.bfloat16)
        dwa = 0.15 * torch.randn(i + 2, generator=g)
        dwa[-1] += 1.0
        W[p + "dwa"] = dwa.to(torch.bfloat16)
        mp = p + "mix."
        H = m["heads"]
        D, DV = m["dim"], m.get("vdim", m["dim"])
        if layer["type"] == "channel_delta":
            G, K = m.get("kv_heads", H), m["conv"]
            ra, rg = ranks
            lin(mp + "q", G * D, width, 2.0)
            lin(mp + "k", G * D, width, 2.0)
            lin(mp + "v", H * DV, width, 2.0)
            for n, c in (("q", G * D), ("k", G * D), ("v", H * DV)):
                W[mp + n + ".conv"] = (
                    0.6 * torch.randn(c, K, generator=g)).to(torch.bfloat16)
            lin(mp + "b", H, width, 2.0)
            lin(mp + "a1", ra, width, 2.0)
            lin(mp + "a2", H * D, ra, 2.0)
            vec(mp + "dt_bias", H * D, -1.0, 1.0)
            vec(mp + "A_log", H, -0.5, 0.7)
            lin(mp + "g1", rg, width, 2.0)
            lin(mp + "g2", H * DV, rg, 2.0)
            vec(mp + "norm", DV, 1.0, 0.2)
            lin(mp + "o", width, H * DV)
        elif layer["type"] == "attention":
            G = m.get("kv_heads", H)
            lin(mp + "q", H * D, width, 2.0)
            lin(mp + "k", G * D, width, 2.0)
            lin(mp + "v", G * DV, width)
            vec(mp + "q.b", H * D, 0.0, 0.3)
            vec(mp + "k.b", G * D, 0.0, 0.3)
            vec(mp + "v.b", G * DV, 0.0, 0.3)
            # strong head-norm weights: scores spread, so window edges and
            # the cap matter
            vec(mp + "q.norm", D, 1.5, 0.5)
            vec(mp + "k.norm", D, 1.5, 0.5)
            W[mp + "vmix"] = torch.tensor(0.35 + 0.1 * i).to(torch.bfloat16)
            vec(mp + "sink", H, 0.5, 1.0)
            lin(mp + "o", width, H * DV)
        else:
            R, L = m["rot_dim"], m["kv_rank"]
            lin(mp + "q", H * (D + R), width, 3.0)
            lin(mp + "dkv", L + R, width, 3.0)
            vec(mp + "dkv.norm", L, 1.0, 0.2)
            lin(mp + "uk", H * D, L, 2.0)
            lin(mp + "uv", H * DV, L)
            vec(mp + "sink", H, 0.5, 1.0)
            lin(mp + "o", width, H * DV)
        f = layer.get("mlp")
        if f is not None:
            vec(p + "norm2", width, 1.0, 0.1)
            lin(p + "mlp.gate", f["ff"], width, 2.5)
            lin(p + "mlp.up", f["ff"], width, 2.5)
            lin(p + "mlp.down", width, f["ff"])
    return W
