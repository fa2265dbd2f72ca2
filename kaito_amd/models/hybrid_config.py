"""Per-layer specifications for hybrid stacks (recurrent + windowed
attention layers mixed in one model) and the config.json reader of the
Gurapel design.

A homogeneous model is described by the flat ModelConfig fields; a hybrid
one additionally carries `layer_specs`, one LayerSpec per layer, each
naming its token mixer(s) and its feed-forward. The mixer specs are plain
frozen dataclasses so another design can reuse any of them with its own
constants.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from ..engine.config import ModelConfig


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Gated delta-rule linear attention (matrix-valued recurrent state
    per head, short causal convolutions on q/k/v)."""
    heads: int            # value heads (one state matrix each)
    qk_heads: int         # query/key heads, shared by heads // qk_heads
    dim: int              # per-head query/key size
    vdim: int             # per-head value size
    conv_taps: int        # short-convolution length
    qk_eps: float = 1e-6  # inside the unit-norm root


@dataclass(frozen=True)
class WindowAttnSpec:
    """Softmax attention over a sliding window of the paged cache with
    per-head qk RMS norm, tanh score capping and a logarithmic distance
    penalty instead of a rotation."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int           # a query sees itself and window-1 earlier keys
    scale: float
    softcap: float        # 0 = no capping
    distance_bias: bool = True
    qk_norm: bool = True


@dataclass(frozen=True)
class RGLRUSpec:
    """Recurrent block around a real-gated linear recurrent unit: a GELU
    gate branch beside a conv + diagonal-recurrence branch."""
    width: int
    blocks: int           # block-diagonal gate matrices
    conv_taps: int
    decay_scale: float = 8.0


@dataclass(frozen=True)
class MoESpec:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class LayerSpec:
    # "delta": one DeltaRuleSpec; "parallel": WindowAttnSpec beside
    # RGLRUSpec, outputs normed and averaged
    kind: str
    delta: Optional[DeltaRuleSpec] = None
    attn: Optional[WindowAttnSpec] = None
    rglru: Optional[RGLRUSpec] = None
    moe: Optional[MoESpec] = None     # None = no feed-forward


def _moe_spec(m) -> Optional[MoESpec]:
    if m is None:
        return None
    if m.get("kind", "moe") != "moe":
        raise ValueError(f"unsupported feed-forward kind {m.get('kind')!r}")
    return MoESpec(experts=int(m["router"]["experts"]),
                   top=int(m["router"]["top"]), ff=int(m["expert"]["ff"]))


def _layer_spec(entry: dict) -> LayerSpec:
    kind = entry["type"]
    mx = entry["mixer"]
    moe = _moe_spec(entry.get("mlp"))
    if kind == "delta":
        return LayerSpec(kind, delta=DeltaRuleSpec(
            heads=int(mx["heads"]), qk_heads=int(mx["kv_heads"]),
            dim=int(mx["dim"]), vdim=int(mx["vdim"]),
            conv_taps=int(mx["conv"])), moe=moe)
    if kind == "parallel":
        lf, rt = mx["left"], mx["right"]
        return LayerSpec(
            kind,
            attn=WindowAttnSpec(
                heads=int(lf["heads"]), kv_heads=int(lf["kv_heads"]),
                dim=int(lf["dim"]), vdim=int(lf["vdim"]),
                window=int(lf["mask"]["size"]), scale=float(lf["scale"]),
                softcap=float(lf.get("softcap", 0.0))),
            rglru=RGLRUSpec(width=int(rt["width"]), blocks=int(rt["blocks"]),
                            conv_taps=int(rt["conv"])),
            moe=moe)
    raise ValueError(f"unknown layer type {kind!r}")


def is_gurapel_config(cfg: dict) -> bool:
    return cfg.get("architecture") == "Gurapel"


def gurapel_model_config(cfg: dict, name: str = "",
                         dtype: torch.dtype = torch.bfloat16) -> ModelConfig:
    """config.json of a Gurapel checkpoint → ModelConfig. Every size and
    per-model constant comes from the file; the flat llama-style fields
    are filled with the first attention/MoE layer's numbers only so that
    generic consumers (memory estimator, metrics) see sensible values."""
    specs: Tuple[LayerSpec, ...] = tuple(_layer_spec(e) for e in cfg["layers"])
    width = int(cfg["width"])
    attn = next((s.attn for s in specs if s.attn is not None), None)
    moe = next((s.moe for s in specs if s.moe is not None), None)
    return ModelConfig(
        name=name or "gurapel", arch="gurapel", layer_specs=specs,
        hidden_size=width, num_layers=len(specs),
        num_heads=attn.heads if attn else 1,
        num_kv_heads=attn.kv_heads if attn else 1,
        head_dim=attn.dim if attn else width,
        intermediate_size=moe.ff if moe else width,
        vocab_size=int(cfg["vocab"]),
        max_position=int(cfg["max_positions"]),
        rms_eps=float(cfg["norm"]["eps"]),
        embed_scale=float(cfg["embedding"]["scale"]),
        rms_norm_offset=True, learned_positions=True, residual_fp32=True,
        num_experts=moe.experts if moe else 0,
        num_experts_per_tok=moe.top if moe else 0,
        moe_intermediate_size=moe.ff if moe else 0,
        moe_routing="topk_softmax", dtype=dtype)


def layer_moe_config(cfg: ModelConfig, moe: MoESpec) -> ModelConfig:
    """A per-layer view of cfg for MoEMLP (layers may differ in expert
    count, top-k and width). For bf16 the expert width is rounded up to
    the 64-column tile of the fused grouped-GEMM kernels (which also keeps
    the vectorised activation kernel's alignment on the per-expert path);
    the loader zero-fills the extra gate/up rows and down columns, which
    contribute exactly nothing (silu(0)·0 = 0)."""
    ff = moe.ff
    if cfg.dtype == torch.bfloat16:
        ff = (ff + 63) // 64 * 64
    return dataclasses.replace(
        cfg, num_experts=moe.experts, num_experts_per_tok=moe.top,
        moe_intermediate_size=ff, moe_routing="topk_softmax",
        moe_act="silu", moe_bias=False, n_shared_experts=0,
        moe_router_fp32=True)
