"""Pokulorn: a pre-norm hybrid decoder stack served by the paged engine.

Every layer is  x ← x + mixer(rms(x)·w₁);  x ← x + ff(rms(x)·w₂)  (the
second half only where the layer has a feed-forward). The stream x is
f32; sub-layers see its norm rounded to the activation dtype. Layer kinds
(models/hybrid_config.py LayerSpec):

  * "mlstm":     MLSTMMixer
  * "attention": RotaryWindowAttention with window + kept first tokens,
                 sink, value mixing across layers
  * "parallel":  RotaryWindowAttention (causal, output gate) beside
                 SSDMixer on the same input, summed with fixed weights

The feed-forward is ClampedGLU. Input: the token embedding; no position
table (positions enter through rotations and masks). Mixer state lives in
the engine's caches: attention K/V in pages; recurrent state and
convolution tails in per-sequence slots.

Each sub-layer's residual add is fused with the NEXT sub-layer's norm
(ops.residual_add_norm), so a layer receives its normed input and is told
the weight of the norm that follows it.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..engine.config import ModelConfig
from .hybrid_base import HybridStackBase, MixerLayerBase, f32_vector
from .hybrid_config import LayerSpec
from .mixers import ClampedGLU, MLSTMMixer, RotaryWindowAttention, SSDMixer


class PokulornLayer(MixerLayerBase):
    def __init__(self, cfg: ModelConfig, spec: LayerSpec):
        super().__init__()
        self.cfg, self.spec = cfg, spec
        h, eps, dt = cfg.hidden_size, cfg.rms_eps, cfg.dtype
        self.attn = self.ssd = self.mixer = None
        if spec.kind == "mlstm":
            self.mixer = MLSTMMixer(h, spec.mlstm, dt, eps)
        elif spec.kind == "attention":
            self.attn = RotaryWindowAttention(h, spec.rattn, dt, eps)
        elif spec.kind == "parallel":
            self.attn = RotaryWindowAttention(h, spec.rattn, dt, eps)
            self.ssd = SSDMixer(h, spec.ssd, dt, eps)
        else:
            raise ValueError(spec.kind)
        self.norm1 = f32_vector(h)
        if spec.dense is not None:
            self.mlp = ClampedGLU(h, spec.dense, dt)
            self.norm2 = f32_vector(h)
        else:
            self.mlp = None

    def mixers(self):
        return [m for m in (self.mixer, self.attn, self.ssd) if m is not None]

    def forward(self, x32, h, positions, cache, meta, next_norm):
        """h = rms(x32)·norm1 in the activation dtype. Returns the next
        layer's normed input (None after the last layer)."""
        eps, dt = self.cfg.rms_eps, self.cfg.dtype
        after_mixer = self.norm2 if self.mlp is not None else next_norm
        if self.spec.kind == "parallel":
            ya = self.attn(h, positions, self._view(cache, self.attn), meta)
            ys = self.ssd(h, positions, self._view(cache, self.ssd), meta)
            s1, s2 = self.spec.branch_scales
            h = ops.residual_add_norm(x32, ya, after_mixer, eps, dt, y2=ys,
                                      s1=s1, s2=s2)
        else:
            m = self.mixer if self.mixer is not None else self.attn
            y = m(h, positions, self._view(cache, m), meta)
            h = ops.residual_add_norm(x32, y, after_mixer, eps, dt)
        if self.mlp is not None:
            h = ops.residual_add_norm(x32, self.mlp(h), next_norm, eps, dt)
        return h


class PokulornForCausalLM(HybridStackBase):
    def __init__(self, cfg: ModelConfig):
        super().__init__(cfg)
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size,
                                         dtype=cfg.dtype)
        self.embed_tokens.weight.requires_grad_(False)
        self.layers = nn.ModuleList(
            [PokulornLayer(cfg, s) for s in cfg.layer_specs])
        self.norm = f32_vector(cfg.hidden_size)
        self.lm_head = nn.Parameter(
            torch.empty(cfg.vocab_size, cfg.hidden_size, dtype=cfg.dtype),
            requires_grad=False)

    def decode_graph_capturable(self) -> bool:
        """No decode-step op of this stack reads device data on the host."""
        return True

    def forward(self, input_ids, positions, kv_caches, meta,
                hidden_in=None) -> torch.Tensor:
        cfg = self.cfg
        meta.layer_shared = {}
        x32 = self.embed_tokens(input_ids).float()
        h = ops.rms_norm_cast(x32, self.layers[0].norm1, cfg.rms_eps,
                              cfg.dtype)
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < n else None
            h = layer(x32, h, positions, kv_caches[i], meta, nxt)
            if self.layer_hook is not None:
                self.layer_hook(i, x32)
        return x32

    # ---- weights ----------------------------------------------------------
    @torch.no_grad()
    def random_init(self, seed: int = 0):
        """Random weights of the right shapes with magnitudes that keep
        every mechanism active (decays away from 0 and 1, gates open)."""
        dev = self.lm_head.device
        gen = torch.Generator(device=dev).manual_seed(seed)

        def normal(p, std):
            t = torch.empty(p.shape, dtype=torch.float32, device=dev)
            t.normal_(0, std, generator=gen)
            p.copy_(t.to(p.dtype))

        def uniform(p, lo, hi):
            t = torch.empty(p.shape, dtype=torch.float32, device=dev)
            t.uniform_(lo, hi, generator=gen)
            p.copy_(t.to(p.dtype))

        for name, p in self.named_parameters():
            last = name.split(".")[-1]
            if last in ("norm", "norm1", "norm2", "out_norm", "q_norm",
                        "k_norm"):
                uniform(p, 0.8, 1.2)
            elif last in ("conv_bias", "dt_bias", "gate_bias", "sinks"):
                normal(p, 0.5)
            elif last == "conv_weight":
                normal(p, 0.4)
            elif last == "a_log":
                uniform(p, -2.0, 0.5)
            elif last == "d_skip":
                uniform(p, 0.5, 1.5)
            elif "embed" in name:
                normal(p, 0.5)
            else:
                normal(p, 1.0 / math.sqrt(p.shape[-1]))
        k = 0
        for layer in self.layers:
            if layer.attn is not None and layer.attn.spec.mix_values:
                layer.attn.v_lambda = 0.2 + 0.1 * (k % 5)
                k += 1
        return self
