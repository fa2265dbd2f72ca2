"""Gurapel: a hybrid decoder stack served by the paged engine.

Every layer is  x ← x + norm1(mixer(x));  x ← x + norm2(ff(x))  — the
norms sit on the sub-layer OUTPUTS, the sub-layers read the residual
stream itself. The stream is f32; sub-layers see its rounding to the
activation dtype. Layer kinds (models/hybrid_config.py LayerSpec):

  * "delta":    GatedDeltaMixer
  * "parallel": BiasedWindowAttention beside RGLRUMixer on the same input;
                each output is RMS-normed over the model width with its
                own weight and the two are averaged.

The feed-forward is the engine's MoEMLP (top-k on f32 router logits,
softmax over the selected logits). Input: scaled token embedding plus a
learned absolute position vector. Mixer state lives in the engine's
caches: attention K/V in pages, recurrent state in per-sequence slots.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..engine.config import ModelConfig
from .hybrid_base import HybridStackBase, MixerLayerBase
from .hybrid_config import LayerSpec, layer_moe_config
from .mixers import BiasedWindowAttention, GatedDeltaMixer, RGLRUMixer
from .moe import MoEMLP


def _vec(n):
    return nn.Parameter(torch.empty(n, dtype=torch.float32),
                        requires_grad=False)


class HybridLayer(MixerLayerBase):
    def __init__(self, cfg: ModelConfig, spec: LayerSpec):
        super().__init__()
        self.cfg, self.spec = cfg, spec
        h, eps = cfg.hidden_size, cfg.rms_eps
        if spec.kind == "delta":
            self.mixer = GatedDeltaMixer(h, spec.delta, cfg.dtype, eps)
        elif spec.kind == "parallel":
            self.attn = BiasedWindowAttention(h, spec.attn, cfg.dtype, eps)
            self.rglru = RGLRUMixer(h, spec.rglru, cfg.dtype)
            self.attn_out_norm = _vec(h)     # plain weights
            self.rglru_out_norm = _vec(h)
        else:
            raise ValueError(spec.kind)
        # output norms hold 1 + w (folded at load)
        self.norm1 = _vec(h)
        if spec.moe is not None:
            self.mlp = MoEMLP(layer_moe_config(cfg, spec.moe))
            self.norm2 = _vec(h)
        else:
            self.mlp = None

    def mixers(self):
        return [self.mixer] if self.spec.kind == "delta" else \
            [self.attn, self.rglru]

    def forward(self, x32, xa, positions, cache, meta):
        cfg = self.cfg
        eps, dt = cfg.rms_eps, cfg.dtype
        if self.spec.kind == "delta":
            y = self.mixer(xa, positions, self._view(cache, self.mixer), meta)
            xa = ops.post_norm_residual(x32, y, self.norm1, eps, dt)
        else:
            ya = self.attn(xa, positions, self._view(cache, self.attn), meta)
            yr = self.rglru(xa, positions, self._view(cache, self.rglru), meta)
            xa = ops.post_norm_residual(x32, ya, self.norm1, eps, dt, y2=yr,
                                        w_y=self.attn_out_norm,
                                        w_y2=self.rglru_out_norm)
        if self.mlp is not None:
            f = self.mlp(xa)
            xa = ops.post_norm_residual(x32, f, self.norm2, eps, dt)
        return xa


class GurapelForCausalLM(HybridStackBase):
    def __init__(self, cfg: ModelConfig):
        super().__init__(cfg)
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size,
                                         dtype=cfg.dtype)
        self.embed_tokens.weight.requires_grad_(False)
        self.pos_embed = nn.Parameter(
            torch.empty(cfg.max_position, cfg.hidden_size, dtype=cfg.dtype),
            requires_grad=False)
        self.layers = nn.ModuleList(
            [HybridLayer(cfg, s) for s in cfg.layer_specs])
        self.norm = _vec(cfg.hidden_size)            # 1 + w
        self.lm_head = nn.Parameter(
            torch.empty(cfg.vocab_size, cfg.hidden_size, dtype=cfg.dtype),
            requires_grad=False)

    # ---- engine interface -------------------------------------------------
    def decode_graph_capturable(self) -> bool:
        """True when no decode-step op reads device data on the host: the
        MoE layers must take the fused grouped-GEMM path (bf16, 64-aligned
        width and padded expert width)."""
        return all(
            layer.mlp is None or (
                self.cfg.dtype == torch.bfloat16
                and self.cfg.hidden_size % 64 == 0
                and layer.mlp.ie_local % 64 == 0)
            for layer in self.layers)

    def forward(self, input_ids, positions, kv_caches, meta,
                hidden_in=None) -> torch.Tensor:
        cfg = self.cfg
        x32 = self.embed_tokens(input_ids).float() * cfg.embed_scale \
            + self.pos_embed[positions].float()
        xa = x32 if cfg.dtype == torch.float32 else x32.to(cfg.dtype)
        for i, layer in enumerate(self.layers):
            xa = layer(x32, xa, positions, kv_caches[i], meta)
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
            if last in ("norm", "norm1", "norm2", "attn_out_norm",
                        "rglru_out_norm", "out_norm", "q_norm", "k_norm"):
                uniform(p, 0.8, 1.2)
            elif last in ("in_bias", "conv_bias", "gate_b", "dt_bias"):
                normal(p, 0.1)
            elif last == "conv_weight":
                normal(p, 0.4)
            elif last == "a_log":
                uniform(p, -1.5, 0.5)
            elif last == "decay_rate":
                uniform(p, 0.05, 1.0)
            elif last == "r1":
                uniform(p, 0.1, 1.0)
            elif last == "r2":
                uniform(p, 0.1, 2.0)
            elif last in ("embed_tokens", "pos_embed") or "embed" in name:
                normal(p, 0.5)
            else:
                fan_in = p.shape[-1] if last != "gate_w" else p.shape[-2]
                normal(p, 1.0 / math.sqrt(fan_in))
        return self
