"""Token mixers for heterogeneous (per-layer spec) models.

Each mixer exposes
  * in_params(): its input-projection parameters, so a layer can run ONE
                GEMM over [mixer rows | feed-forward rows] of the shared
                norm output;
  * cache_shape(): what the runner must allocate per layer — a paged KV
                pair for attention, a per-sequence fp32 state for the
                recurrence;
  * forward_from_proj(proj, meta, cache) -> the mixer's pre-output-projection
                activations [T, out_in], and out_weight [width, out_in].
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from production_stack_amd import ops
from production_stack_amd.engine.config import MixerSpec
from production_stack_amd.ops import gemm_policy

# decay = exp(-DECAY_SCALE * sigmoid(.)): the per-step decay stays in
# (exp(-DECAY_SCALE), 1)
DELTA_DECAY_SCALE = math.exp(-0.5)


class TalkAttention(nn.Module):
    """Grouped-query softmax attention over the paged KV cache with the
    MixerSpec's options: no rotary code, score mixing across heads,
    aligned-chunk / trailing-window visibility, denominator sink; key and
    value widths may differ."""

    kind = "attention"

    def __init__(self, width: int, spec: MixerSpec,
                 dtype: torch.dtype) -> None:
        super().__init__()
        if spec.rope:
            raise NotImplementedError(
                "TalkAttention carries no rotary code; rope layers use the "
                "Llama attention path")
        self.spec = spec
        H, G = spec.heads, spec.kv_heads or spec.heads
        D, DV = spec.dim, spec.vdim or spec.dim
        if H % G:
            raise ValueError("heads must be a multiple of kv_heads")
        self.H, self.G, self.D, self.DV = H, G, D, DV
        self.qkv = nn.Parameter(
            torch.empty(H * D + G * D + G * DV, width, dtype=dtype))
        self.out_weight = nn.Parameter(
            torch.empty(width, H * DV, dtype=dtype))
        self.talk = (
            nn.Parameter(torch.empty(H, H, dtype=torch.float32))
            if spec.talking_heads else None)
        self.scale = spec.scale or 1.0 / math.sqrt(D)

    def in_params(self):
        return [self.qkv]

    @property
    def out_in(self) -> int:
        return self.H * self.DV

    def cache_shape(self):
        return ("kv", self.G, self.D, self.DV)

    def forward_from_proj(self, proj: torch.Tensor, meta, cache,
                          out: Optional[torch.Tensor] = None
                          ) -> torch.Tensor:
        H, G, D, DV = self.H, self.G, self.D, self.DV
        k_cache, v_cache = cache
        q = proj[:, :H * D]
        k = proj[:, H * D:H * D + G * D]
        v = proj[:, H * D + G * D:]
        ops.kv_append(k, v, k_cache, v_cache, meta.slot_mapping)
        sp = self.spec
        T = proj.shape[0]
        if out is None:
            out = torch.empty((T, H * DV), dtype=proj.dtype,
                              device=proj.device)
        # batch rows: multi-token prompt portions first, single tokens
        # after them. Portions share key tiles between neighbouring rows
        # (tiled kernel); single tokens of different sequences share
        # nothing and take the split-key kernel, one workgroup per token.
        npt = min(getattr(meta, "num_prefill_tokens", T) or 0, T)
        for a, b, variant in ((0, npt, 0), (npt, T, 3)):
            if b > a:
                ops.talk_attention(
                    q[a:b], k_cache, v_cache, meta.block_tables,
                    meta.token_seq[a:b], meta.positions[a:b], self.scale, H,
                    chunk=sp.chunk, window=sp.window, sink=sp.sink,
                    talk=self.talk, out=out[a:b], variant=variant)
        return out


class GeneralDelta(nn.Module):
    """Gated delta-rule linear recurrence ("generalized delta rule"): per
    head a dim x dim fp32 state with a per-channel data-dependent decay
    (low-rank projection) and a per-channel removal gate along the unit
    key; the read-out is RMS-normalised per head, channel-scaled and
    gated. State lives in a per-sequence slot of the runner's state
    cache."""

    kind = "general_delta"

    def __init__(self, width: int, spec: MixerSpec, eps: float,
                 dtype: torch.dtype) -> None:
        super().__init__()
        self.spec = spec
        self.eps = eps
        H, D, R = spec.heads, spec.dim, spec.decay_rank
        self.H, self.D, self.R = H, D, R
        HD = H * D
        # fused rows: r | k | v | g | a | w1
        self.in_proj = nn.Parameter(torch.empty(5 * HD + R, width,
                                                dtype=dtype))
        self.w2 = nn.Parameter(torch.empty(HD, R, dtype=dtype))
        self.w0 = nn.Parameter(torch.empty(HD, dtype=torch.float32))
        self.a_bias = nn.Parameter(torch.empty(HD, dtype=torch.float32))
        self.out_norm = nn.Parameter(torch.empty(HD, dtype=torch.float32))
        self.out_weight = nn.Parameter(torch.empty(width, HD, dtype=dtype))

    def in_params(self):
        return [self.in_proj]

    @property
    def out_in(self) -> int:
        return self.H * self.D

    def cache_shape(self):
        return ("state", self.H, self.D, self.D)

    def forward_from_proj(self, proj: torch.Tensor, meta, cache,
                          out: Optional[torch.Tensor] = None
                          ) -> torch.Tensor:
        HD = self.H * self.D
        r = proj[:, 0:HD]
        k = proj[:, HD:2 * HD]
        v = proj[:, 2 * HD:3 * HD]
        g = proj[:, 3 * HD:4 * HD]
        za = proj[:, 4 * HD:5 * HD]
        zw = gemm_policy.linear(torch.tanh(proj[:, 5 * HD:]), self.w2)
        return ops.delta_rule(
            r, k, v, zw, za, g, self.w0, self.a_bias, self.out_norm, cache,
            meta.seq_rows, self.H, self.eps, DELTA_DECAY_SCALE, out=out)


def build_mixer(width: int, spec: MixerSpec, eps: float,
                dtype: torch.dtype) -> nn.Module:
    if spec.kind == "attention":
        return TalkAttention(width, spec, dtype)
    if spec.kind == "general_delta":
        return GeneralDelta(width, spec, eps, dtype)
    raise ValueError(f"unknown mixer kind {spec.kind!r}")
