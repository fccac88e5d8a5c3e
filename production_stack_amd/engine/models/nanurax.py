"""Nanurax: a hybrid decoder — gated delta-rule recurrent layers interleaved
with chunk-masked, head-mixed attention layers; dense or routed
feed-forwards; one norm per layer feeding mixer and feed-forward in
parallel.

Numerics: the residual stream is fp32 end to end (embedding, per-layer sum,
norms); norms, router, attention scores/weights and everything inside the
recurrence are fp32; projections and their activations run in the serving
dtype (bfloat16, or float32 for an all-fp32 engine).

Per layer the GPU work is
    [fused add + RMSNorm]  ->  ONE GEMM over [mixer rows | feed-forward rows]
    -> mixer kernel, activation kernel
    -> dense layers: ONE GEMM over [mixer out | ff act] x [W_o | W_down]
       routed layers: W_o GEMM + expert GEMMs, summed in fp32.

config.json layout read here: architecture, vocab, width, norm.eps,
embedding.scale, layers[i] = {type, mixer{...}, mlp{...}|null}.
Checkpoint names: embed, head, final.norm, l<i>.norm1, l<i>.mix.*,
l<i>.mlp.* (experts e<j>, shared expert "shared").
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
from production_stack_amd.engine.models.ffn import GatedMLP, SparseMoE
from production_stack_amd.engine.models.mixers import build_mixer
from production_stack_amd.ops import gemm_policy

ARCHITECTURE = "Nanurax"


# ---------------------------------------------------------------------------
# configuration
# ---------------------------------------------------------------------------
def _mixer_spec(kind: str, m: dict, decay_rank: int = 0) -> MixerSpec:
    if kind == "attention":
        mask = m.get("mask") or {}
        return MixerSpec(
            kind="attention", heads=m["heads"], dim=m["dim"],
            kv_heads=m.get("kv_heads", m["heads"]),
            vdim=m.get("vdim", m["dim"]), scale=m["scale"],
            chunk=int(mask.get("size", 0)), window=0, sink=True,
            talking_heads=True, rope=False)
    if kind == "general_delta":
        return MixerSpec(kind="general_delta", heads=m["heads"],
                         dim=m["dim"], rope=False, decay_rank=decay_rank)
    raise ValueError(f"unknown layer type {kind!r}")


def _mlp_spec(m: Optional[dict]) -> Optional[MlpSpec]:
    if m is None:
        return None
    if m["kind"] == "dense":
        return MlpSpec(kind="dense", ff=m["ff"], act="gelu_tanh")
    if m["kind"] == "moe":
        shared = m.get("shared") or {}
        return MlpSpec(
            kind="moe", ff=m["expert"]["ff"], act="clamped_swish",
            limit=float(m["expert"]["limit"]),
            experts=m["router"]["experts"], top=m["router"]["top"],
            score="sigmoid", renormalize=False, weight_on_input=True,
            shared_ff=int(shared.get("ff", 0)),
            shared_limit=float(shared.get("limit", 0.0)))
    raise ValueError(f"unknown mlp kind {m['kind']!r}")


def config_from_json(cfg: dict, name: str = "nanurax",
                     decay_ranks: Optional[dict] = None) -> ModelConfig:
    """decay_ranks: layer index -> rank of the low-rank decay projection
    (a tensor shape, not a config.json entry; the checkpoint reader passes
    it in, named configs carry it as mixer.decay_rank)."""
    specs: List[LayerSpec] = []
    for i, layer in enumerate(cfg["layers"]):
        m = layer["mixer"]
        rank = (decay_ranks or {}).get(i, m.get("decay_rank", 0))
        specs.append(LayerSpec(
            mixer=_mixer_spec(layer["type"], m, rank),
            mlp=_mlp_spec(layer.get("mlp")), parallel=True))
    att = [s.mixer for s in specs if s.mixer.kind == "attention"]
    ffs = [s.mlp.ff for s in specs if s.mlp is not None]
    return ModelConfig(
        name=name, family="nanurax", hidden_size=cfg["width"],
        num_layers=len(specs),
        num_q_heads=max([m.heads for m in att], default=1),
        num_kv_heads=max([m.kv_heads for m in att], default=1),
        head_dim=max([m.dim for m in att], default=1),
        intermediate_size=max(ffs, default=0), vocab_size=cfg["vocab"],
        max_position=1 << 20, rms_norm_eps=float(cfg["norm"]["eps"]),
        layer_specs=specs,
        embedding_scale=float(cfg["embedding"]["scale"]),
        # no BOS/EOS convention in this design: never stop on a token id
        bos_token_id=0, eos_token_id=-1)


def config_from_dir(path: str) -> ModelConfig:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    ranks = {}
    st = os.path.join(path, "model.safetensors")
    if os.path.exists(st):
        from production_stack_amd.engine.weights import safetensors_header

        for key, info in safetensors_header(st).items():
            parts = key.split(".")
            if len(parts) == 3 and parts[1:] == ["mix", "w1"]:
                ranks[int(parts[0][1:])] = int(info["shape"][0])
    return config_from_json(cfg, name=os.path.basename(
        os.path.normpath(path)) or "nanurax", decay_ranks=ranks)


# ---------------------------------------------------------------------------
# model
# ---------------------------------------------------------------------------
class NanuraxLayer(nn.Module):
    def __init__(self, width: int, spec: LayerSpec, eps: float,
                 dtype: torch.dtype) -> None:
        super().__init__()
        if not spec.parallel:
            raise NotImplementedError("sequential sublayers")
        self.spec = spec
        self.eps = eps
        self.norm = nn.Parameter(torch.empty(width, dtype=torch.float32))
        self.mixer = build_mixer(width, spec.mixer, eps, dtype)
        self.mlp = None
        if spec.mlp is not None:
            if spec.mlp.kind == "dense":
                self.mlp = GatedMLP(width, spec.mlp.ff, spec.mlp.act,
                                    spec.mlp.limit, dtype)
            else:
                self.mlp = SparseMoE(width, spec.mlp, dtype)
        self.w_in = None   # fused [mixer rows | ff rows], built by fuse()
        self.w_out = None  # dense layers: fused [W_o | W_down]

    @torch.no_grad()
    def fuse(self) -> None:
        """Build the fused projection weights from the loaded parts; the
        input-side parts become views of the fused buffer."""
        parts = list(self.mixer.in_params())
        self.mix_rows = sum(p.shape[0] for p in parts)
        if self.mlp is not None:
            parts += list(self.mlp.in_params())
        self.w_in = torch.cat([p.data for p in parts], dim=0).contiguous()
        off = 0
        for p in parts:
            p.data = self.w_in[off:off + p.shape[0]]
            off += p.shape[0]
        if isinstance(self.mlp, GatedMLP):
            self.w_out = torch.cat(
                [self.mixer.out_weight.data, self.mlp.down.data],
                dim=1).contiguous()

    def forward(self, h: torch.Tensor, meta, cache) -> List[torch.Tensor]:
        """h: normed input [T, width]. Returns the deltas that join the
        residual stream (summed in fp32 by the next fused add+norm)."""
        if self.w_in is None:
            self.fuse()
        proj = gemm_policy.linear(h, self.w_in)
        mproj = proj[:, :self.mix_rows]
        fproj = proj[:, self.mix_rows:]
        if self.w_out is not None:
            # dense: both branches write into one buffer, one out GEMM
            mo, ff = self.mixer.out_in, self.mlp.ff
            cat = torch.empty((h.shape[0], mo + ff), dtype=h.dtype,
                              device=h.device)
            self.mixer.forward_from_proj(mproj, meta, cache,
                                         out=cat[:, :mo])
            self.mlp.inner(fproj, out=cat[:, mo:])
            return [gemm_policy.linear(cat, self.w_out)]
        mix = self.mixer.forward_from_proj(mproj, meta, cache)
        deltas = [gemm_policy.linear(mix, self.mixer.out_weight)]
        if self.mlp is not None:
            # routed feed-forward: fp32 sum of experts (+ shared), rounded
            # once to the serving dtype
            deltas.append(self.mlp.forward_from_proj(
                h, fproj if fproj.shape[1] else None).to(h.dtype))
        return deltas


class NanuraxForCausalLM(nn.Module):
    # per-step metadata this family needs from the runner
    needs_seq_meta = True
    supports_decode_graph = False

    def __init__(self, cfg: ModelConfig, tp: int = 1, pp_rank: int = 0,
                 pp_size: int = 1, dtype: torch.dtype = torch.bfloat16
                 ) -> None:
        super().__init__()
        if tp != 1 or pp_size != 1:
            raise NotImplementedError(
                "Nanurax runs on one GPU per replica (no TP/PP sharding of "
                "the recurrent state yet)")
        self.cfg = cfg
        self.tp = 1
        self.dtype = dtype
        W = cfg.hidden_size
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                              dtype=dtype))
        self.layers = nn.ModuleList(
            NanuraxLayer(W, spec, cfg.rms_norm_eps, dtype)
            for spec in cfg.layer_specs)
        self.final_norm = nn.Parameter(torch.empty(W, dtype=torch.float32))
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                                dtype=dtype))
        # optional debugging tap: called with (layer index, fp32 residual
        # stream after that layer)
        self.residual_hook = None

    # ---- cache geometry ------------------------------------------------
    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def cache_shapes(self):
        return [layer.mixer.cache_shape() for layer in self.layers]

    def kv_bytes_per_block(self, block_size: int) -> int:
        esz = 4 if self.dtype == torch.float32 else 2
        return sum(
            g * block_size * (d + dv) * esz
            for kind, g, d, dv in self.cache_shapes() if kind == "kv")

    def state_bytes_per_seq(self) -> int:
        return sum(h * d * dv * 4
                   for kind, h, d, dv in self.cache_shapes()
                   if kind == "state")

    def gemm_weights(self):
        """One weight per distinct projection shape of the stack (for the
        per-shape GEMM choice at decode batch sizes)."""
        seen, out = set(), []
        for layer in self.layers:
            if layer.w_in is None:
                layer.fuse()
            cands = [layer.w_in, layer.w_out, layer.mixer.out_weight]
            if hasattr(layer.mixer, "w2"):
                cands.append(layer.mixer.w2)
            if isinstance(layer.mlp, SparseMoE) and layer.mlp.shared:
                cands.append(layer.mlp.shared.down)
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
            if name.endswith("norm"):
                p.normal_(1.0, 0.1, generator=gen)
            elif name.endswith(("w0", "a_bias")):
                p.normal_(0.0, 0.5, generator=gen)
            elif name.endswith("talk"):
                p.normal_(0.0, 0.2, generator=gen)
                p.add_(torch.eye(p.shape[0], device=dev, dtype=p.dtype))
            else:
                p.normal_(0.0, p.shape[-1] ** -0.5, generator=gen)
        for layer in self.layers:
            layer.w_in = layer.w_out = None

    @torch.no_grad()
    def load_weights(self, path: str) -> None:
        from safetensors import safe_open

        f = safe_open(os.path.join(path, "model.safetensors"),
                      framework="pt", device="cpu")

        def put(param, name):
            t = f.get_tensor(name)
            if tuple(t.shape) != tuple(param.shape):
                raise ValueError(
                    f"{name}: checkpoint shape {tuple(t.shape)} != "
                    f"{tuple(param.shape)}")
            param.copy_(t.to(param.dtype))

        def cat(names):
            return torch.cat([f.get_tensor(n) for n in names], dim=0)

        put(self.embed, "embed")
        put(self.lm_head, "head")
        put(self.final_norm, "final.norm")
        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            put(layer.norm, pre + "norm1")
            mx, mp = layer.mixer, pre + "mix."
            if mx.kind == "attention":
                mx.qkv.copy_(cat([mp + "q", mp + "k", mp + "v"]).to(
                    mx.qkv.dtype))
                put(mx.out_weight, mp + "o")
                if mx.talk is not None:
                    put(mx.talk, mp + "talk")
            else:
                mx.in_proj.copy_(cat(
                    [mp + n for n in ("r", "k", "v", "g", "a", "w1")]
                ).to(mx.in_proj.dtype))
                put(mx.w2, mp + "w2")
                put(mx.w0, mp + "w0")
                put(mx.a_bias, mp + "a.b")
                put(mx.out_norm, mp + "norm")
                put(mx.out_weight, mp + "o")
            ml, lp = layer.mlp, pre + "mlp."
            if isinstance(ml, GatedMLP):
                ml.gate_up.copy_(cat([lp + "gate", lp + "up"]).to(
                    ml.gate_up.dtype))
                put(ml.down, lp + "down")
            elif isinstance(ml, SparseMoE):
                put(ml.router, lp + "router")
                for e in range(ml.spec.experts):
                    ep = f"{lp}e{e}."
                    ml.experts_gate_up[e].copy_(
                        cat([ep + "gate", ep + "up"]).to(
                            ml.experts_gate_up.dtype))
                    ml.experts_down[e].copy_(
                        f.get_tensor(ep + "down").to(ml.experts_down.dtype))
                if ml.shared is not None:
                    sp = lp + "shared."
                    ml.shared.gate_up.copy_(
                        cat([sp + "gate", sp + "up"]).to(
                            ml.shared.gate_up.dtype))
                    put(ml.shared.down, sp + "down")
                    put(ml.shared_gate, sp + "sg")
            layer.w_in = layer.w_out = None

    def _apply(self, fn, *a, **kw):
        # fused weights are plain tensors rebuilt lazily after a move/cast
        for layer in self.layers:
            layer.w_in = layer.w_out = None
        return super()._apply(fn, *a, **kw)

    # ---- forward -------------------------------------------------------
    @torch.no_grad()
    def forward(self, token_ids: torch.Tensor, meta, caches,
                residual=None) -> torch.Tensor:
        cfg = self.cfg
        x = ops.embed_scale(token_ids, self.embed, cfg.embedding_scale)
        deltas: List[torch.Tensor] = []
        hook = self.residual_hook
        for i, (layer, cache) in enumerate(zip(self.layers, caches)):
            h = ops.add_rms_norm32(x, deltas, layer.norm, cfg.rms_norm_eps,
                                   self.dtype)
            if hook is not None and i > 0:
                hook(i - 1, x)
            deltas = layer(h, meta, cache)
        h = ops.add_rms_norm32(x, deltas, self.final_norm,
                               cfg.rms_norm_eps, self.dtype)
        if hook is not None:
            hook(len(self.layers) - 1, x)
        return h

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.lm_head).float()
