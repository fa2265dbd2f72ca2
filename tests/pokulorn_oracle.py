"""Plain restatement of the Pokulorn design for tests: float64 numpy, token
loops, one function per mechanism, operating on checkpoint-named tensors.
Nothing here is shared with the package; it exists to be obviously right,
not fast.

Notation: h is a sub-layer's input row, W[name] a checkpoint tensor
(linear maps stored [out, in]), rms(v) = v / sqrt(mean(v^2) + eps).
"""
from __future__ import annotations

import math

import numpy as np


def rms(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def short_conv(u, w, bias=None):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t-taps+1+j), zeros
    before the sequence."""
    T, C = u.shape
    taps = w.shape[1]
    pad = np.concatenate([np.zeros((taps - 1, C)), u], 0)
    y = np.zeros((T, C))
    for t in range(T):
        for j in range(taps):
            y[t] += w[:, j] * pad[t + j]
    if bias is not None:
        y = y + bias
    return y


def rotary_tables(rot, positions):
    """cos, sin [T, dims/2] with the interpolated frequencies and the
    magnitude factor of the length extension (when given)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    freq = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def turn_dim(t):
            return dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))
        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        ramp = np.clip((np.arange(half) - lo) / max(hi - lo, 0.001), 0, 1)
        freq = freq / factor * ramp + freq * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freq[None, :]
    return np.cos(ang) * mag, np.sin(ang) * mag


def rotate(x, cos, sin):
    """x [T, heads, dim]; the first 2*half dims rotate, i paired with
    i + half."""
    half = cos.shape[1]
    out = x.copy()
    a, b = x[..., :half], x[..., half:2 * half]
    c, s = cos[:, None, :], sin[:, None, :]
    out[..., :half] = a * c - b * s
    out[..., half:2 * half] = b * c + a * s
    return out


def attention(h, W, pre, mx, eps, v_first=None, mix_values=False,
              sink=True, gate=False):
    """Softmax attention with short convolutions, per-head q/k norm,
    partial rotation, an optional window that keeps the first tokens, an
    optional sink in the denominator, optional mixing with another
    layer's values and an optional sigmoid output gate. Returns
    (out [T, width], values as cached [T, G*vdim])."""
    T = h.shape[0]
    H, G, D, V = (int(mx[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    q = short_conv(h @ W[pre + "q"].T, W[pre + "q.conv"])
    k = short_conv(h @ W[pre + "k"].T, W[pre + "k.conv"])
    v = short_conv(h @ W[pre + "v"].T, W[pre + "v.conv"])
    q = rms(q.reshape(T, H, D), eps) * W[pre + "q.norm"]
    k = rms(k.reshape(T, G, D), eps) * W[pre + "k.norm"]
    cos, sin = rotary_tables(mx["rot"], np.arange(T))
    q, k = rotate(q, cos, sin), rotate(k, cos, sin)
    if mix_values and v_first is not None:
        lam = float(W[pre + "vmix"])
        v = (1 - lam) * v + lam * v_first
    vh = v.reshape(T, G, V)
    mask = mx.get("mask")
    out = np.zeros((T, H, V))
    for i in range(T):
        if mask:
            js = [j for j in range(i + 1)
                  if i - j < int(mask["size"]) or j < int(mask["keep_first"])]
        else:
            js = list(range(i + 1))
        for hd in range(H):
            g = hd // (H // G)
            s = np.array([q[i, hd] @ k[j, g] for j in js]) * float(mx["scale"])
            top = s.max()
            if sink:
                top = max(top, float(W[pre + "sink"][hd]))
            e = np.exp(s - top)
            den = e.sum()
            if sink:
                den += math.exp(float(W[pre + "sink"][hd]) - top)
            out[i, hd] = (e / den) @ vh[js, g]
    o = out.reshape(T, H * V)
    if gate:
        o = o * sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T, v


def mlstm(h, W, pre, mx, eps):
    """Matrix memory with exponential input gate, stabilised by a running
    maximum that starts at 0."""
    T = h.shape[0]
    H, D, V = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
    cap = float(mx["gate_cap"])
    q = (h @ W[pre + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ W[pre + "k"].T).reshape(T, H, D)
    v = (h @ W[pre + "v"].T).reshape(T, H, V)
    gi = cap * np.tanh((h @ W[pre + "i"].T + W[pre + "i.b"]) / cap)
    gf = log_sigmoid(cap * np.tanh((h @ W[pre + "f"].T + W[pre + "f.b"]) / cap))
    o = np.zeros((T, H, V))
    for hd in range(H):
        S = np.zeros((D, V))
        n = np.zeros(D)
        m = 0.0
        for t in range(T):
            m_new = max(gf[t, hd] + m, gi[t, hd])
            keep = math.exp(gf[t, hd] + m - m_new)
            take = math.exp(gi[t, hd] - m_new)
            S = keep * S + take * np.outer(k[t, hd], v[t, hd])
            n = keep * n + take * k[t, hd]
            m = m_new
            den = max(abs(n @ q[t, hd]), math.exp(-m)) + 1e-6
            o[t, hd] = (S.T @ q[t, hd]) / den
    o = rms(o, eps).reshape(T, H * V) * W[pre + "norm"]
    o = o * sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def ssd(h, W, pre, mx, eps):
    """Selective state space with a scalar decay per head and step."""
    T = h.shape[0]
    H, P, N, G = (int(mx[k]) for k in ("heads", "vdim", "state", "groups"))
    parts = int(mx["norm_groups"])
    inner = H * P
    p = h @ W[pre + "in"].T
    z = p[:, :inner]
    xbc = p[:, inner:2 * inner + 2 * G * N]
    dt = p[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, W[pre + "conv"], W[pre + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + W[pre + "dt_bias"])
    rate = np.exp(W[pre + "A_log"])
    y = np.zeros((T, H, P))
    for hd in range(H):
        g = hd // (H // G)
        S = np.zeros((N, P))
        for t in range(T):
            S = math.exp(-rate[hd] * dt[t, hd]) * S \
                + dt[t, hd] * np.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + W[pre + "D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner)
    return (y * W[pre + "norm"]) @ W[pre + "o"].T


def feed_forward(h, W, pre, ff):
    lim = float(ff["limit"])
    g = np.minimum(h @ W[pre + "gate"].T, lim)
    u = np.clip(h @ W[pre + "up"].T, -lim, lim)
    return (g * sigmoid(1.702 * g) * (u + 1)) @ W[pre + "down"].T


def forward(cfg, W, tokens, streams=None):
    """Logits [T, vocab] of one sequence; `streams`, a list, receives the
    residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][np.asarray(tokens)]
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        pre, mx = f"l{i}.", layer["mixer"]
        h = rms(x, eps) * W[pre + "norm1"]
        kind = layer["type"]
        if kind == "mlstm":
            y = mlstm(h, W, pre + "mix.", mx, eps)
        elif kind == "attention":
            mixes = bool(mx.get("v_mix"))
            y, v = attention(h, W, pre + "mix.", mx, eps, v_first=v_first,
                             mix_values=mixes, sink=True, gate=False)
            if mixes and v_first is None:
                v_first = v
        elif kind == "parallel":
            left, _ = attention(h, W, pre + "mix.left.", mx["left"], eps,
                                sink=False, gate=True)
            right = ssd(h, W, pre + "mix.right.", mx["right"], eps)
            y = float(mx["left_scale"]) * left + float(mx["right_scale"]) * right
        else:
            raise ValueError(kind)
        x = x + y
        if layer.get("mlp"):
            h = rms(x, eps) * W[pre + "norm2"]
            x = x + feed_forward(h, W, pre + "mlp.", layer["mlp"])
        if streams is not None:
            streams.append(x.copy())
    return (rms(x, eps) * W["final.norm"]) @ W["head"].T


# ---- configurations and random checkpoints for tests ---------------------

def mlstm_layer(heads, dim, vdim, gate_cap=10.0, mlp=None):
    return {"type": "mlstm", "mlp": mlp, "mixer": {
        "heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}}


def rot(dims, base=10000.0, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"),
                                scaling))
    return r


def attention_mixer(heads, kv_heads, dim, vdim, conv, rot_, scale,
                    window=None, keep_first=0, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "conv": conv, "rot": rot_, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window, "keep_first": keep_first}
    if v_mix:
        m["v_mix"] = True
    return m


def attention_layer(mlp=None, **kw):
    return {"type": "attention", "mlp": mlp, "mixer": attention_mixer(**kw)}


def parallel_layer(left, heads, vdim, state, groups, norm_groups, conv,
                   left_scale=0.5, right_scale=0.5, mlp=None):
    return {"type": "parallel", "mlp": mlp, "mixer": {
        "left": left, "left_scale": left_scale, "right_scale": right_scale,
        "right": {"heads": heads, "vdim": vdim, "state": state,
                  "groups": groups, "norm_groups": norm_groups,
                  "conv": conv}}}


def dense(ff, limit=4.0):
    return {"kind": "dense", "ff": ff, "limit": limit}


def make_config(layers, width, vocab, eps=1e-5):
    return {"architecture": "Pokulorn", "layers": layers,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_weights(cfg, seed=0, slow_decay=False):
    """bf16-representable random tensors under the checkpoint's names, as
    float64 numpy arrays. slow_decay keeps the recurrent memories long
    (forget gates near 1, small state-space steps) so that far-away
    tokens still matter."""
    import torch
    gen = torch.Generator().manual_seed(seed)
    W = {}

    def rnd(name, *shape, std=1.0, mean=0.0):
        t = torch.randn(*shape, generator=gen) * std + mean
        W[name] = t.to(torch.bfloat16).double().numpy()

    width = cfg["width"]
    rnd("embed", cfg["vocab"], width)
    rnd("final.norm", width, std=0.2, mean=1.0)
    rnd("head", cfg["vocab"], width, std=width ** -0.5)

    def attention_weights(q, a, gate, sink):
        nq, nk, nv = (a["heads"] * a["dim"], a["kv_heads"] * a["dim"],
                      a["kv_heads"] * a["vdim"])
        for n, rows in (("q", nq), ("k", nk), ("v", nv)):
            rnd(q + n, rows, width, std=width ** -0.5)
            rnd(q + n + ".conv", rows, a["conv"], std=0.6)
        rnd(q + "q.norm", a["dim"], std=0.3, mean=1.0)
        rnd(q + "k.norm", a["dim"], std=0.3, mean=1.0)
        if sink:
            rnd(q + "sink", a["heads"], std=1.0)
        if a.get("v_mix"):
            W[q + "vmix"] = np.float64(
                torch.rand((), generator=gen).to(torch.bfloat16).item())
        if gate:
            rnd(q + "g", a["heads"] * a["vdim"], width, std=width ** -0.5)
        rnd(q + "o", width, a["heads"] * a["vdim"],
            std=(a["heads"] * a["vdim"]) ** -0.5)

    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        rnd(p + "norm1", width, std=0.2, mean=1.0)
        m = L["mixer"]
        if L["type"] == "mlstm":
            q = p + "mix."
            nqk, nv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            rnd(q + "q", nqk, width, std=width ** -0.5)
            rnd(q + "k", nqk, width, std=width ** -0.5)
            rnd(q + "v", nv, width, std=width ** -0.5)
            rnd(q + "g", nv, width, std=width ** -0.5)
            rnd(q + "i", m["heads"], width, std=2 * width ** -0.5)
            rnd(q + "i.b", m["heads"], std=0.5)
            rnd(q + "f", m["heads"], width, std=2 * width ** -0.5)
            rnd(q + "f.b", m["heads"], std=0.5,
                mean=6.0 if slow_decay else 2.0)
            rnd(q + "norm", nv, std=0.3, mean=1.0)
            rnd(q + "o", width, nv, std=nv ** -0.5)
        elif L["type"] == "attention":
            attention_weights(p + "mix.", m, gate=False, sink=True)
        else:
            attention_weights(p + "mix.left.", m["left"], gate=True,
                              sink=False)
            r, q = m["right"], p + "mix.right."
            inner = r["heads"] * r["vdim"]
            ch = inner + 2 * r["groups"] * r["state"]
            rnd(q + "in", inner + ch + r["heads"], width, std=width ** -0.5)
            rnd(q + "conv", ch, r["conv"], std=0.6)
            rnd(q + "conv.b", ch, std=0.2)
            rnd(q + "dt_bias", r["heads"], std=0.5,
                mean=-4.0 if slow_decay else -1.0)
            rnd(q + "A_log", r["heads"], std=0.5,
                mean=-3.0 if slow_decay else 0.0)
            rnd(q + "D", r["heads"], std=0.5, mean=1.0)
            rnd(q + "norm", inner, std=0.3, mean=1.0)
            rnd(q + "o", width, inner, std=inner ** -0.5)
        if L.get("mlp") is not None:
            q, ff = p + "mlp.", L["mlp"]["ff"]
            rnd(p + "norm2", width, std=0.2, mean=1.0)
            rnd(q + "gate", ff, width, std=2 * width ** -0.5)
            rnd(q + "up", ff, width, std=2 * width ** -0.5)
            rnd(q + "down", width, ff, std=ff ** -0.5)
    return W


def write_checkpoint(folder, cfg, W):
    import json
    import os

    import torch
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: torch.tensor(np.asarray(v)).to(torch.bfloat16).contiguous()
               for k, v in W.items()},
              os.path.join(folder, "model.safetensors"))
    return folder


def model_logits(cfg, W, tokens, streams=None):
    """forward() as a float64 torch tensor (streams likewise)."""
    import torch
    st = [] if streams is not None else None
    out = torch.from_numpy(forward(cfg, W, tokens, st))
    if streams is not None:
        streams.extend(torch.from_numpy(s) for s in st)
    return out
