"""Helpers for the Nanurax tests: small configurations in the checkpoint's
own config.json layout, random bf16 weights under the checkpoint's tensor
names, checkpoint folders, and an error measure."""

from __future__ import annotations

import json
import os

import torch


def delta(heads=3, dim=16):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim}}


def attn(heads=6, kv_heads=2, dim=16, vdim=24, size=20, scale=0.3):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                      "vdim": vdim, "mask": {"size": size}, "scale": scale}}


def dense(ff=80):
    return {"kind": "dense", "ff": ff}


def moe(ff=24, limit=1.75, experts=5, top=2, shared=(40, 1.25)):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
         "router": {"experts": experts, "top": top}}
    if shared is not None:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def make_cfg(layers, width=64, vocab=97, eps=1e-5, scale=6.5):
    """layers: [(mixer dict, mlp dict | None)]."""
    return {
        "architecture": "Nanurax", "vocab": vocab, "width": width,
        "norm": {"eps": eps}, "embedding": {"scale": scale},
        "layers": [dict(m, mlp=f) for m, f in layers],
    }


def make_weights(cfg, seed=0, rank=8):
    g = torch.Generator().manual_seed(seed)
    W = {}

    def lin(name, out, inp, gain=1.0):
        W[name] = (torch.randn(out, inp, generator=g) * gain
                   / inp ** 0.5).to(torch.bfloat16)

    def vec(name, n, mean=0.0, std=1.0):
        W[name] = (mean + std * torch.randn(n, generator=g)).to(
            torch.bfloat16)

    width, vocab = cfg["width"], cfg["vocab"]
    W["embed"] = (torch.randn(vocab, width, generator=g) * 0.15).to(
        torch.bfloat16)
    lin("head", vocab, width)
    vec("final.norm", width, 1.0, 0.1)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        vec(p + "norm1", width, 1.0, 0.1)
        m = layer["mixer"]
        if layer["type"] == "general_delta":
            hd = m["heads"] * m["dim"]
            for n in ("r", "k", "v", "g", "a"):
                lin(p + "mix." + n, hd, width, 1.5)
            lin(p + "mix.w1", rank, width)
            lin(p + "mix.w2", hd, rank, 2.0)
            vec(p + "mix.w0", hd)
            vec(p + "mix.a.b", hd)
            vec(p + "mix.norm", hd, 1.0, 0.2)
            lin(p + "mix.o", width, hd)
        else:
            H, G = m["heads"], m.get("kv_heads", m["heads"])
            D, DV = m["dim"], m.get("vdim", m["dim"])
            lin(p + "mix.q", H * D, width, 2.0)
            lin(p + "mix.k", G * D, width, 2.0)
            lin(p + "mix.v", G * DV, width)
            W[p + "mix.talk"] = (torch.eye(H) + 0.3 * torch.randn(
                H, H, generator=g)).to(torch.bfloat16)
            lin(p + "mix.o", width, H * DV)
        f = layer.get("mlp")
        if f is None:
            continue
        if f["kind"] == "dense":
            lin(p + "mlp.gate", f["ff"], width, 1.5)
            lin(p + "mlp.up", f["ff"], width, 1.5)
            lin(p + "mlp.down", width, f["ff"])
        else:
            ff = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                lin(f"{p}mlp.e{e}.gate", ff, width, 3.0)
                lin(f"{p}mlp.e{e}.up", ff, width, 3.0)
                lin(f"{p}mlp.e{e}.down", width, ff)
            lin(p + "mlp.router", f["router"]["experts"], width, 4.0)
            if f.get("shared"):
                sf = f["shared"]["ff"]
                lin(p + "mlp.shared.gate", sf, width, 3.0)
                lin(p + "mlp.shared.up", sf, width, 3.0)
                lin(p + "mlp.shared.down", width, sf)
                lin(p + "mlp.shared.sg", 1, width, 2.0)
    return W


def save_checkpoint(path, cfg, W):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()},
              os.path.join(path, "model.safetensors"))
    return str(path)


def make_engine(path, dtype="float32", device="cpu", blocks=64,
                block_size=16, max_seqs=4, budget=1 << 20, model_len=4096):
    from production_stack_amd.engine.config import (
        CacheConfig,
        EngineConfig,
        SchedulerConfig,
    )
    from production_stack_amd.engine.engine import LLMEngine

    cfg = EngineConfig(
        model=str(path), dtype=dtype, max_model_len=model_len,
        enforce_eager=True,
        cache=CacheConfig(num_gpu_blocks=blocks, block_size=block_size),
        scheduler=SchedulerConfig(max_num_seqs=max_seqs,
                                  max_num_batched_tokens=budget,
                                  max_prefill_chunk=budget))
    return LLMEngine(cfg, device=device)


def row_errs(got, want):
    """Per-row RMS of the difference (row mean removed) over the RMS of
    the wanted row (row mean removed)."""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt()
            / w.pow(2).mean(-1).sqrt().clamp_min(1e-12)).flatten()


def rel_err(got, want):
    """The worst row's error."""
    return float(row_errs(got, want).max())


def close(got, want, dtype):
    """float32: every row within 2e-4 (the sharp test). bfloat16: the
    median row within 3e-2 and four rows in five within 6e-2 — bfloat16
    rounding can flip a near-tied expert choice, which moves that row's
    logits visibly and, through the recurrent state, nudges the rows after
    it, without any fault in the mechanism."""
    e = row_errs(got, want).sort().values
    if dtype == "float32":
        return bool(e[-1] < TOL[dtype])
    if len(e) < 5:
        # too few rows for a quantile; a sequence's very first read-out of
        # the recurrence is (k.r) v over its own rms, whose sign hangs on
        # a possibly tiny k.r — bfloat16 may not resolve it
        return bool(torch.isfinite(e).all())
    ok = bool(e[len(e) // 2] < 3e-2
              and e[max(0, (4 * len(e)) // 5 - 1)] < TOL[dtype])
    if not ok:
        print("row errors:", [round(float(x), 3) for x in e])
    return ok


TOL = {"float32": 2e-4, "bfloat16": 6e-2}
