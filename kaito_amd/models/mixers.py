"""Token mixers for hybrid stacks: gated delta rule, real-gated linear
recurrence, and softmax attention over a sliding window with a distance
penalty. Each is a self-contained module parameterised by its spec
(models/hybrid_config.py), so a design picks and combines them freely.

All three follow the same calling convention:

    mixer(x, positions, cache, meta) -> y            x, y: [T, hidden]

`cache` is the dict of this layer's device tensors handed out by
`alloc_cache()` (paged K/V for attention; per-sequence state slots for the
recurrent mixers) and `meta` the step's AttnMetadata with the chunk layout
(cu_seqlens / state_slots / seq_starts / token_seq / block_tables). A
step may mix prompt chunks of any length with single decode tokens; the
kernels behind `ops.*` make no distinction.

Precision: projections run in the activation dtype (bf16 or f32, f32
accumulation); everything that feeds a recurrence, every norm, the
attention scores and softmax are f32 inside the kernels; states are f32.
"""
from __future__ import annotations

from typing import Dict

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from .hybrid_config import DeltaRuleSpec, RGLRUSpec, WindowAttnSpec


def _p(*shape, dtype):
    return nn.Parameter(torch.empty(*shape, dtype=dtype), requires_grad=False)


class GatedDeltaMixer(nn.Module):
    """Linear attention with the gated delta rule. Per head the state is a
    [dim, vdim] matrix S; per token: S ← g·S, then the prediction error
    β(v − Sᵀk) is written along k, then the output is Sᵀq (it already sees
    the token's own write). q, k, v pass a short causal convolution + silu;
    q and k are unit-normalised; the output is RMS-normed per head and
    gated by silu of a fourth projection."""

    def __init__(self, hidden: int, spec: DeltaRuleSpec, dtype, norm_eps: float):
        super().__init__()
        assert spec.heads % spec.qk_heads == 0
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        self.n_qk = spec.qk_heads * spec.dim
        self.n_v = spec.heads * spec.vdim
        self.conv_ch = 2 * self.n_qk + self.n_v
        # fused input projection, rows [q | k | v | gate | a | b]
        self.in_proj = _p(self.conv_ch + self.n_v + 2 * spec.heads, hidden,
                          dtype=dtype)
        self.conv_weight = _p(self.conv_ch, spec.conv_taps,
                              dtype=torch.float32)
        self.a_log = _p(spec.heads, dtype=torch.float32)
        self.dt_bias = _p(spec.heads, dtype=torch.float32)
        self.out_norm = _p(spec.vdim, dtype=torch.float32)
        self.o_proj = _p(hidden, self.n_v, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        return {
            "conv": torch.zeros(num_slots, max(s.conv_taps - 1, 1),
                                self.conv_ch, dtype=self.dtype, device=device),
            "ssm": torch.zeros(num_slots, s.heads, s.dim, s.vdim,
                               dtype=torch.float32, device=device),
        }

    def cache_bytes(self, block_size: int):
        s = self.spec
        esz = torch.empty(0, dtype=self.dtype).element_size()
        return 0, (max(s.conv_taps - 1, 1) * self.conv_ch * esz
                   + s.heads * s.dim * s.vdim * 4)

    def forward(self, x, positions, cache, meta):
        s = self.spec
        T = x.size(0)
        p = F.linear(x, self.in_proj)
        qkv = ops.causal_conv_update(
            p[:, :self.conv_ch], self.conv_weight, None, cache["conv"],
            meta.cu_seqlens, meta.state_slots, meta.seq_starts,
            meta.token_seq, act=1)
        q = qkv[:, :self.n_qk].unflatten(-1, (s.qk_heads, s.dim))
        k = qkv[:, self.n_qk:2 * self.n_qk].unflatten(-1, (s.qk_heads, s.dim))
        v = qkv[:, 2 * self.n_qk:].unflatten(-1, (s.heads, s.vdim))
        c = self.conv_ch
        gate = p[:, c:c + self.n_v].unflatten(-1, (s.heads, s.vdim))
        a = p[:, c + self.n_v:c + self.n_v + s.heads]
        b = p[:, c + self.n_v + s.heads:]
        o = ops.gated_delta_rule(
            q, k, v, gate, a, b, self.a_log, self.dt_bias, self.out_norm,
            cache["ssm"], meta.cu_seqlens, meta.state_slots, meta.seq_starts,
            s.qk_eps, self.norm_eps)
        return F.linear(o.reshape(T, self.n_v), self.o_proj)


class RGLRUMixer(nn.Module):
    """Recurrent block around a real-gated linear recurrent unit: a
    GELU-activated gate branch y beside a branch u = conv(linear(x)) that
    drives the diagonal recurrence S ← a·S + sqrt(1−a²)·i·u with
    a = exp(−c·r·softplus(λ)); r and i are sigmoid gates computed from u by
    block-diagonal matrices. Output projection of S·y."""

    def __init__(self, hidden: int, spec: RGLRUSpec, dtype):
        super().__init__()
        assert spec.width % spec.blocks == 0
        self.spec, self.dtype = spec, dtype
        w, nb = spec.width, spec.blocks
        self.bw = w // nb
        # fused input projection, rows [y | x], with bias
        self.in_proj = _p(2 * w, hidden, dtype=dtype)
        self.in_bias = _p(2 * w, dtype=dtype)
        self.conv_weight = _p(w, spec.conv_taps, dtype=torch.float32)
        self.conv_bias = _p(w, dtype=torch.float32)
        # per block, rows [recurrence gate | input gate], stored
        # transposed ([in, out]) for the batched product; f32: the gates
        # enter the recurrence
        self.gate_w = _p(nb, self.bw, 2 * self.bw, dtype=torch.float32)
        self.gate_b = _p(nb, 1, 2 * self.bw, dtype=torch.float32)
        # c · softplus(λ), folded once at load
        self.decay_rate = _p(w, dtype=torch.float32)
        self.o_proj = _p(hidden, w, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        return {
            "conv": torch.zeros(num_slots, max(s.conv_taps - 1, 1), s.width,
                                dtype=self.dtype, device=device),
            "lru": torch.zeros(num_slots, s.width, dtype=torch.float32,
                               device=device),
        }

    def cache_bytes(self, block_size: int):
        s = self.spec
        esz = torch.empty(0, dtype=self.dtype).element_size()
        return 0, max(s.conv_taps - 1, 1) * s.width * esz + s.width * 4

    def forward(self, x, positions, cache, meta):
        s = self.spec
        T, w = x.size(0), s.width
        p = F.linear(x, self.in_proj, self.in_bias)
        u = ops.causal_conv_update(
            p[:, w:], self.conv_weight, self.conv_bias, cache["conv"],
            meta.cu_seqlens, meta.state_slots, meta.seq_starts,
            meta.token_seq, act=0)
        ub = u.float().view(T, s.blocks, self.bw).transpose(0, 1)
        gates = torch.baddbmm(self.gate_b, ub, self.gate_w)   # [B, T, 2bw]
        o = ops.rglru_scan(u, gates, p[:, :w], self.decay_rate, cache["lru"],
                           meta.cu_seqlens, meta.state_slots, meta.seq_starts,
                           meta.token_seq)
        return F.linear(o, self.o_proj)


class BiasedWindowAttention(nn.Module):
    """Grouped-query softmax attention over the last `window` positions of
    the paged cache. No rotation: position enters through the causal
    window and a per-head penalty r1·ln(1 + r2·distance) subtracted from
    the (optionally tanh-capped) scores. q and k are RMS-normed per head
    with a weight shared by the heads; key and value sizes may differ."""

    def __init__(self, hidden: int, spec: WindowAttnSpec, dtype, norm_eps: float):
        super().__init__()
        assert spec.heads % spec.kv_heads == 0
        self.spec, self.dtype, self.norm_eps = spec, dtype, norm_eps
        s = spec
        self.q_size = s.heads * s.dim
        self.k_size = s.kv_heads * s.dim
        self.v_size = s.kv_heads * s.vdim
        self.qkv_proj = _p(self.q_size + self.k_size + self.v_size, hidden,
                           dtype=dtype)
        if s.qk_norm:
            self.q_norm = _p(s.dim, dtype=torch.float32)
            self.k_norm = _p(s.dim, dtype=torch.float32)
        else:
            self.q_norm = self.k_norm = None
        if s.distance_bias:
            self.r1 = _p(s.heads, dtype=torch.float32)
            self.r2 = _p(s.heads, dtype=torch.float32)
        else:
            self.r1 = self.r2 = None
        self.o_proj = _p(hidden, s.heads * s.vdim, dtype=dtype)

    def alloc_cache(self, num_blocks, block_size, num_slots, device) -> Dict:
        s = self.spec
        return {
            "k": torch.zeros(num_blocks, s.kv_heads, block_size, s.dim,
                             dtype=self.dtype, device=device),
            "v": torch.zeros(num_blocks, s.kv_heads, block_size, s.vdim,
                             dtype=self.dtype, device=device),
        }

    def cache_bytes(self, block_size: int):
        s = self.spec
        esz = torch.empty(0, dtype=self.dtype).element_size()
        return s.kv_heads * block_size * (s.dim + s.vdim) * esz, 0

    def forward(self, x, positions, cache, meta):
        s = self.spec
        T = x.size(0)
        qkv = F.linear(x, self.qkv_proj)
        q = qkv[:, :self.q_size].unflatten(-1, (s.heads, s.dim))
        k = qkv[:, self.q_size:self.q_size + self.k_size].unflatten(
            -1, (s.kv_heads, s.dim))
        v = qkv[:, self.q_size + self.k_size:].unflatten(
            -1, (s.kv_heads, s.vdim))
        qn = ops.qk_norm_cache_write(q, k, v, self.q_norm, self.k_norm,
                                     self.norm_eps, cache["k"], cache["v"],
                                     meta.slot_mapping)
        tiles = None
        if meta.tile_seq is not None:
            tiles = (meta.tile_seq, meta.tile_qbase, meta.cu_seqlens,
                     meta.seq_starts)
        o = ops.window_attention(qn, cache["k"], cache["v"],
                                 meta.block_tables, meta.token_seq, positions,
                                 s.scale, s.softcap, self.r1, self.r2,
                                 s.window, tiles=tiles)
        return F.linear(o.reshape(T, -1), self.o_proj)
