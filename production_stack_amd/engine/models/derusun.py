"""Derusun: a hybrid decoder of sequential pre-norm layers whose mixers are
channel-decay gated delta-rule recurrences, sliding-window attention with
kept first keys, or latent attention; every layer reads a token-shifted
norm output and hands on a learned weighted sum of all streams so far.

Per layer i, with x the stream the previous layer handed on:
    h  = shift(groupnorm(x) * w1)      shift: h_t + (h_{t-1} - h_t) * mu
    x' = x + mixer(h)
    x' = x' + ff(groupnorm(x') * w2)   (layers with a feed-forward)
    X_{i+1} = x';  handed on: sum_{j <= i+1} dwa_i[j] * X_j   (X_0 = embedding)
The output is the grouped norm of the last handed-on stream times the head.

Numerics: the streams X_j, their sums and all norms are fp32; attention
scores/weights and everything inside the recurrence are fp32 (in the
kernels); projections, convolutions and activations run in the serving
dtype (bfloat16, or float32 for an all-fp32 engine).

Per layer the GPU work is
    fused grouped norm + token shift (state: previous token's normed row)
    ONE GEMM over all of the mixer's input projections
    mixer kernels (conv + recurrence | norm/blend/append + attention |
                   latent norm/rotary/append + attention)
    W_o GEMM; fused residual add + grouped norm; gate|up GEMM; activation;
    W_down GEMM; fused residual add + depth-weighted sum.

config.json layout read here: architecture, vocab, width, norm{eps, groups},
layers[i] = {type, mixer{...}, mlp{kind, ff, limit}|null}.
Checkpoint names: embed, head, final.norm, l<i>.norm1/norm2/shift/dwa,
l<i>.mix.*, l<i>.mlp.gate/up/down.
"""

from __future__ import annotations

import json
import os
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from production_stack_amd import ops
from production_stack_amd.engine.config import (
    LayerSpec,
    MixerSpec,
    MlpSpec,
    ModelConfig,
)
from production_stack_amd.engine.models.ffn import GatedMLP
from production_stack_amd.engine.models.mixers import build_mixer
from production_stack_amd.ops import gemm_policy

ARCHITECTURE = "Derusun"

# positions a rotary table is built for unless the engine asks for more
DEFAULT_MAX_POSITION = 8192


# ---------------------------------------------------------------------------
# configuration
# ---------------------------------------------------------------------------
def _mixer_spec(kind: str, m: dict, ranks: dict) -> MixerSpec:
    if kind == "attention":
        mask = m.get("mask") or {}
        return MixerSpec(
            kind="attention", heads=m["heads"], dim=m["dim"],
            kv_heads=m.get("kv_heads", m["heads"]),
            vdim=m.get("vdim", m["dim"]), scale=float(m["scale"]),
            window=int(mask.get("size", 0)),
            keep_first=int(mask.get("keep_first", 0)),
            softcap=float(m.get("softcap") or 0.0), sink=True,
            learned_sink=True, bias=True, qk_norm=True,
            v_mix=bool(m.get("v_mix", False)), rope=False)
    if kind == "latent_attention":
        rot = m.get("rot") or {}
        return MixerSpec(
            kind="latent_attention", heads=m["heads"], dim=m["dim"],
            kv_heads=1, vdim=m.get("vdim", m["dim"]),
            scale=float(m["scale"]), kv_rank=m["kv_rank"],
            rot_dim=m["rot_dim"],
            rot_dims=int(rot.get("dims", m["rot_dim"])),
            rot_base=float(rot.get("base", 10000.0)), sink=True,
            learned_sink=True, rope=True)
    if kind == "channel_delta":
        return MixerSpec(
            kind="channel_delta", heads=m["heads"], dim=m["dim"],
            kv_heads=m.get("kv_heads", m["heads"]),
            vdim=m.get("vdim", m["dim"]), conv=int(m.get("conv", 1)),
            decay_rank=int(ranks.get("a1", m.get("decay_rank", 0))),
            gate_rank=int(ranks.get("g1", m.get("gate_rank", 0))),
            rope=False)
    raise ValueError(f"unknown layer type {kind!r}")


def _mlp_spec(m: Optional[dict]) -> Optional[MlpSpec]:
    if m is None:
        return None
    if m["kind"] == "dense":
        return MlpSpec(kind="dense", ff=m["ff"], act="clamped_swish",
                       limit=float(m["limit"]))
    raise ValueError(f"unknown mlp kind {m['kind']!r}")


def config_from_json(cfg: dict, name: str = "derusun",
                     ranks: Optional[dict] = None) -> ModelConfig:
    """ranks: layer index -> {"a1": rows, "g1": rows} of the low-rank decay
    and gate projections (tensor shapes, not config.json entries; the
    checkpoint reader passes them in, named configs carry them as
    mixer.decay_rank / mixer.gate_rank)."""
    specs: List[LayerSpec] = []
    for i, layer in enumerate(cfg["layers"]):
        specs.append(LayerSpec(
            mixer=_mixer_spec(layer["type"], layer["mixer"],
                              (ranks or {}).get(i, {})),
            mlp=_mlp_spec(layer.get("mlp")), parallel=False,
            token_shift=True, depth_average=True))
    att = [s.mixer for s in specs if s.mixer.kind != "channel_delta"]
    ffs = [s.mlp.ff for s in specs if s.mlp is not None]
    norm = cfg["norm"]
    return ModelConfig(
        name=name, family="derusun", hidden_size=cfg["width"],
        num_layers=len(specs),
        num_q_heads=max([m.heads for m in att], default=1),
        num_kv_heads=max([m.kv_heads for m in att], default=1),
        head_dim=max([m.dim for m in att], default=1),
        intermediate_size=max(ffs, default=0), vocab_size=cfg["vocab"],
        max_position=int(cfg.get("max_position", DEFAULT_MAX_POSITION)),
        rms_norm_eps=float(norm["eps"]),
        norm_groups=int(norm.get("groups", 1)), layer_specs=specs,
        # no BOS/EOS convention in this design: never stop on a token id
        bos_token_id=0, eos_token_id=-1)


def config_from_dir(path: str) -> ModelConfig:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    ranks: dict = {}
    st = os.path.join(path, "model.safetensors")
    if os.path.exists(st):
        from production_stack_amd.engine.weights import safetensors_header

        for key, info in safetensors_header(st).items():
            parts = key.split(".")
            if len(parts) == 3 and parts[1] == "mix" \
                    and parts[2] in ("a1", "g1"):
                ranks.setdefault(int(parts[0][1:]), {})[parts[2]] = int(
                    info["shape"][0])
    return config_from_json(cfg, name=os.path.basename(
        os.path.normpath(path)) or "derusun", ranks=ranks)


# ---------------------------------------------------------------------------
# model
# ---------------------------------------------------------------------------
class DerusunLayer(nn.Module):
    def __init__(self, width: int, index: int, spec: LayerSpec, eps: float,
                 dtype: torch.dtype, max_pos: int) -> None:
        super().__init__()
        if spec.parallel:
            raise NotImplementedError("parallel sublayers")
        self.spec = spec
        f32 = torch.float32
        self.norm1 = nn.Parameter(torch.empty(width, dtype=f32))
        self.shift = (nn.Parameter(torch.empty(width, dtype=f32))
                      if spec.token_shift else None)
        # weights of the embedding output and the results of layers 0..index
        self.dwa = (nn.Parameter(torch.empty(index + 2, dtype=f32))
                    if spec.depth_average else None)
        self.mixer = build_mixer(width, spec.mixer, eps, dtype, max_pos)
        self.mlp = None
        self.norm2 = None
        if spec.mlp is not None:
            self.norm2 = nn.Parameter(torch.empty(width, dtype=f32))
            self.mlp = GatedMLP(width, spec.mlp.ff, spec.mlp.act,
                                spec.mlp.limit, dtype)

    def cache_shape(self, width: int):
        c = self.mixer.cache_shape()
        if self.shift is not None:
            # the previous token's normed row, per sequence
            return ("multi", [c, ("slots", (width,), torch.float32)])
        return ("multi", [c])


class DerusunForCausalLM(nn.Module):
    # per-step metadata this family needs from the runner
    needs_seq_meta = True
    # no data-dependent control flow: single-token steps replay a hipGraph
    supports_decode_graph = True

    def __init__(self, cfg: ModelConfig, tp: int = 1, pp_rank: int = 0,
                 pp_size: int = 1, dtype: torch.dtype = torch.bfloat16
                 ) -> None:
        super().__init__()
        if tp != 1 or pp_size != 1:
            raise NotImplementedError(
                "Derusun runs on one GPU per replica (no TP/PP sharding of "
                "the recurrent state yet)")
        self.cfg = cfg
        self.tp = 1
        self.dtype = dtype
        W = cfg.hidden_size
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                              dtype=dtype))
        self.layers = nn.ModuleList(
            DerusunLayer(W, i, spec, cfg.rms_norm_eps, dtype,
                         cfg.max_position)
            for i, spec in enumerate(cfg.layer_specs))
        self.final_norm = nn.Parameter(torch.empty(W, dtype=torch.float32))
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                                dtype=dtype))
        # optional debugging tap: called with (layer index, fp32 stream the
        # layer hands on)
        self.residual_hook = None

    # ---- cache geometry ------------------------------------------------
    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def cache_shapes(self):
        W = self.cfg.hidden_size
        return [layer.cache_shape(W) for layer in self.layers]

    def _flat_shapes(self):
        def walk(d):
            if d[0] == "multi":
                for c in d[1]:
                    yield from walk(c)
            else:
                yield d
        for d in self.cache_shapes():
            yield from walk(d)

    def kv_bytes_per_block(self, block_size: int) -> int:
        esz = 4 if self.dtype == torch.float32 else 2
        n = 0
        for d in self._flat_shapes():
            if d[0] == "kv":
                n += d[1] * block_size * (d[2] + d[3]) * esz
            elif d[0] == "paged":
                n += d[1] * block_size * d[2] * esz
        return n

    def state_bytes_per_seq(self) -> int:
        esz = 4 if self.dtype == torch.float32 else 2
        n = 0
        for d in self._flat_shapes():
            if d[0] == "state":
                n += d[1] * d[2] * d[3] * 4
            elif d[0] == "slots":
                e = 1
                for s in d[1]:
                    e *= s
                n += e * (4 if d[2] == torch.float32 else esz)
        return n

    def gemm_weights(self):
        """One weight per distinct projection shape of the stack (for the
        per-shape GEMM choice at decode batch sizes)."""
        seen, out = set(), []
        for layer in self.layers:
            mx = layer.mixer
            cands = [getattr(mx, n, None) for n in
                     ("in_proj", "qkv", "a2", "g2", "out_weight")]
            if layer.mlp is not None:
                cands += [layer.mlp.gate_up, layer.mlp.down]
            for w in cands:
                if w is not None and w.dim() == 2 and w.is_contiguous() \
                        and tuple(w.shape) not in seen:
                    seen.add(tuple(w.shape))
                    out.append(w)
        return out

    # ---- weights -------------------------------------------------------
    @torch.no_grad()
    def random_init(self, seed: int = 0) -> None:
        dev = self.embed.device
        gen = torch.Generator(device=dev).manual_seed(seed)
        for name, p in self.named_parameters():
            last = name.rsplit(".", 1)[-1]
            if last in ("norm1", "norm2", "final_norm", "latent_norm",
                        "q_norm", "k_norm", "out_norm"):
                p.normal_(1.0, 0.1, generator=gen)
            elif last == "shift":
                p.uniform_(0.0, 1.0, generator=gen)
            elif last == "dwa":
                # close to "hand on the newest stream"
                p.normal_(0.0, 0.05, generator=gen)
                p[-1] += 1.0
            elif last in ("sink_vals", "dt_bias", "qkv_bias"):
                p.normal_(0.0, 0.5, generator=gen)
            elif last == "a_log":
                p.uniform_(-1.0, 1.0, generator=gen)
            elif last == "vmix":
                p.fill_(0.3)
            else:
                p.normal_(0.0, p.shape[-1] ** -0.5, generator=gen)

    @torch.no_grad()
    def load_weights(self, path: str) -> None:
        from safetensors import safe_open

        f = safe_open(os.path.join(path, "model.safetensors"),
                      framework="pt", device="cpu")

        def put(param, name):
            t = f.get_tensor(name)
            if t.numel() != param.numel() or (
                    t.dim() == param.dim()
                    and tuple(t.shape) != tuple(param.shape)):
                raise ValueError(
                    f"{name}: checkpoint shape {tuple(t.shape)} != "
                    f"{tuple(param.shape)}")
            param.copy_(t.to(param.dtype).view(param.shape))

        def cat(param, names):
            t = torch.cat([f.get_tensor(n) for n in names], dim=0)
            if tuple(t.shape) != tuple(param.shape):
                raise ValueError(
                    f"{names}: checkpoint shape {tuple(t.shape)} != "
                    f"{tuple(param.shape)}")
            param.copy_(t.to(param.dtype))

        put(self.embed, "embed")
        put(self.lm_head, "head")
        put(self.final_norm, "final.norm")
        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            put(layer.norm1, pre + "norm1")
            if layer.shift is not None:
                put(layer.shift, pre + "shift")
            if layer.dwa is not None:
                put(layer.dwa, pre + "dwa")
            mx, mp = layer.mixer, pre + "mix."
            if mx.kind == "attention":
                cat(mx.qkv, [mp + "q", mp + "k", mp + "v"])
                if mx.qkv_bias is not None:
                    cat(mx.qkv_bias, [mp + "q.b", mp + "k.b", mp + "v.b"])
                if mx.q_norm is not None:
                    put(mx.q_norm, mp + "q.norm")
                    put(mx.k_norm, mp + "k.norm")
                if mx.sink_vals is not None:
                    put(mx.sink_vals, mp + "sink")
                if mx.vmix is not None:
                    put(mx.vmix, mp + "vmix")
            elif mx.kind == "latent_attention":
                cat(mx.in_proj, [mp + "q", mp + "dkv"])
                put(mx.latent_norm, mp + "dkv.norm")
                put(mx.uk, mp + "uk")       # [H*dim, L] -> [H, dim, L]
                put(mx.uv, mp + "uv")       # [H*vdim, L] -> [H, vdim, L]
                if mx.sink_vals is not None:
                    put(mx.sink_vals, mp + "sink")
            else:
                cat(mx.in_proj, [mp + n for n in
                                 ("q", "k", "v", "b", "a1", "g1")])
                cat(mx.conv_w, [mp + "q.conv", mp + "k.conv",
                                mp + "v.conv"])
                put(mx.a2, mp + "a2")
                put(mx.g2, mp + "g2")
                put(mx.a_log, mp + "A_log")
                put(mx.dt_bias, mp + "dt_bias")
                put(mx.out_norm, mp + "norm")
            put(mx.out_weight, mp + "o")
            if layer.mlp is not None:
                lp = pre + "mlp."
                put(layer.norm2, pre + "norm2")
                cat(layer.mlp.gate_up, [lp + "gate", lp + "up"])
                put(layer.mlp.down, lp + "down")

    # ---- forward -------------------------------------------------------
    @torch.no_grad()
    def forward(self, token_ids: torch.Tensor, meta, caches,
                residual=None) -> torch.Tensor:
        cfg = self.cfg
        eps, groups, dt = cfg.rms_norm_eps, cfg.norm_groups, self.dtype
        T = token_ids.shape[0]
        cur = ops.embed_scale(token_ids, self.embed, 1.0)     # fp32 [T, W]
        n_layers = len(self.layers)
        hist = None
        if any(layer.dwa is not None for layer in self.layers):
            # every stream so far stays alive for the weighted sums
            hist = torch.empty((n_layers + 1, T, cfg.hidden_size),
                               dtype=torch.float32, device=cur.device)
            hist[0].copy_(cur)
        shared: dict = {}
        hook = self.residual_hook
        for i, (layer, cache) in enumerate(zip(self.layers, caches)):
            if layer.shift is not None:
                h = ops.group_norm_shift(
                    cur, layer.norm1, eps, groups, dt, layer.shift,
                    cache[1], meta.token_seq, meta.seq_rows)
            else:
                h = ops.add_rms_norm32(cur, [], layer.norm1, eps, dt, groups)
            mix = layer.mixer(h, meta, cache[0], shared)
            delta = gemm_policy.linear(mix, layer.mixer.out_weight)
            base = cur
            if layer.mlp is not None:
                # x' = x + mixer output lands in the new stream's place
                base = hist[i + 1] if hist is not None else cur
                h2 = ops.add_rms_norm32(cur, [delta], layer.norm2, eps, dt,
                                        groups, out32=base)
                delta = layer.mlp(h2)
            if layer.dwa is not None:
                cur = ops.depth_mix(hist, i + 2, layer.dwa, base, delta)
            else:
                cur = base + delta.float()
                if hist is not None:
                    hist[i + 1].copy_(cur)
            if hook is not None:
                hook(i, cur)
        return ops.add_rms_norm32(cur, [], self.final_norm, eps, dt, groups)

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.lm_head).float()
