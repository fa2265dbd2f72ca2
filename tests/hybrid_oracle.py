"""Slow, plain re-statement of the hybrid (Gurapel) design's equations, used
as the oracle for the kernels and the engine. float64, one function per
mechanism, token-by-token loops for everything recurrent. Operates directly
on a checkpoint-style dict of tensors (flat names) and the config.json
dict, and shares no code with kaito_amd.

Also builds random checkpoints for the tests.
"""
import json
import math
import os

import torch

F64 = torch.float64


# ---------------------------------------------------------------- pieces

def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi)
                                     * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def short_conv(x, w, bias=None):
    """x [T, C]; w [C, taps], the LAST column weighs the current token."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                out[t] += w[:, j] * x[src]
    if bias is not None:
        out = out + bias
    return out


def delta_rule_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) / math.sqrt(D)
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    step = torch.log1p(torch.exp(h @ W[p + "a"].T + W[p + "dt_bias"]))
    g = torch.exp(-torch.exp(W[p + "A_log"]) * step)
    gate = silu(h @ W[p + "g"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=F64)
    for hd in range(H):
        kv = hd // (H // G)
        S = torch.zeros(D, V, dtype=F64)
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            out[t, hd] = S.T @ q[t, kv]
    out = unit_rms(out, eps) * W[p + "norm"] * gate
    return out.reshape(T, H * V) @ W[p + "o"].T


def window_attention(q, k, v, window, scale, cap, r1, r2):
    """q [T, H, D], k [T, G, D], v [T, G, V] of ONE sequence from its
    first token; query i sees keys j with 0 <= i - j < window."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for hd in range(H):
        kv = hd // (H // G)
        for i in range(T):
            js = [j for j in range(T) if 0 <= i - j < window]
            s = torch.stack([q[i, hd] @ k[j, kv] for j in js]) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            dist = torch.tensor([float(i - j) for j in js], dtype=F64)
            s = s - r1[hd] * torch.log(1 + r2[hd] * dist)
            a = torch.softmax(s, 0)
            out[i, hd] = sum(a[n] * v[j, kv] for n, j in enumerate(js))
    return out


def window_attention_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ W[p + "q"].T).view(T, H, D), eps) * W[p + "q.norm"]
    k = unit_rms((h @ W[p + "k"].T).view(T, G, D), eps) * W[p + "k.norm"]
    v = (h @ W[p + "v"].T).view(T, G, V)
    out = window_attention(q, k, v, m["mask"]["size"], m["scale"],
                           m.get("softcap", 0.0), W[p + "r1"], W[p + "r2"])
    return out.reshape(T, H * V) @ W[p + "o"].T


def rglru_mixer(h, W, p, m):
    T = h.shape[0]
    width, nb = m["width"], m["blocks"]
    bw = width // nb
    y = gelu_tanh(h @ W[p + "y"].T + W[p + "y.b"])
    u = short_conv(h @ W[p + "x"].T + W[p + "x.b"], W[p + "conv"],
                   W[p + "conv.b"])
    r = torch.zeros(T, width, dtype=F64)
    i = torch.zeros(T, width, dtype=F64)
    for b in range(nb):
        ub = u[:, b * bw:(b + 1) * bw]
        r[:, b * bw:(b + 1) * bw] = torch.sigmoid(
            ub @ W[p + "ra"][b].T + W[p + "ra.b"][b])
        i[:, b * bw:(b + 1) * bw] = torch.sigmoid(
            ub @ W[p + "ri"][b].T + W[p + "ri.b"][b])
    a = torch.exp(-8.0 * r * torch.log1p(torch.exp(W[p + "lam"])))
    S = torch.zeros(width, dtype=F64)
    out = torch.zeros(T, width, dtype=F64)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1 - a[t] ** 2) * i[t] * u[t]
        out[t] = S * y[t]
    return out @ W[p + "o"].T


def moe_ff(h, W, p, m):
    top = m["router"]["top"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        z = W[p + "router"] @ h[t]
        idx = torch.argsort(z, descending=True)[:top]
        wts = torch.softmax(z[idx], 0)
        for wt, e in zip(wts, idx.tolist()):
            a = silu(W[f"{p}e{e}.gate"] @ h[t]) * (W[f"{p}e{e}.up"] @ h[t])
            out[t] += wt * (W[f"{p}e{e}.down"] @ a)
    return out


def model_logits(cfg, W, tokens, stream_out=None):
    """All-position logits [T, vocab] of one sequence."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"] \
        + W["pos"][:T]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        if L["type"] == "delta":
            mix = delta_rule_mixer(x, W, p + "mix.", L["mixer"], eps)
        else:
            lf = window_attention_mixer(x, W, p + "mix.left.",
                                        L["mixer"]["left"], eps)
            rt = rglru_mixer(x, W, p + "mix.right.", L["mixer"]["right"])
            mix = 0.5 * (unit_rms(lf, eps) * W[p + "mix.left.out"]
                         + unit_rms(rt, eps) * W[p + "mix.right.out"])
        x = x + unit_rms(mix, eps) * (1 + W[p + "norm1"])
        if L.get("mlp") is not None:
            ff = moe_ff(x, W, p + "mlp.", L["mlp"])
            x = x + unit_rms(ff, eps) * (1 + W[p + "norm2"])
        if stream_out is not None:
            stream_out.append(x.clone())
    x = unit_rms(x, eps) * (1 + W["final.norm"])
    return x @ W["head"].T


# ------------------------------------------------------- random checkpoints

def delta_layer(heads=2, kv_heads=1, dim=16, vdim=24, conv=3, mlp=None):
    return {"type": "delta", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                      "vdim": vdim, "conv": conv}}


def parallel_layer(heads=4, kv_heads=2, dim=16, vdim=8, window=11,
                   scale=0.3, softcap=5.0, width=48, blocks=3, conv=2,
                   mlp=None):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads,
                               "dim": dim, "vdim": vdim,
                               "mask": {"size": window}, "scale": scale,
                               "softcap": softcap},
                      "right": {"width": width, "blocks": blocks,
                                "conv": conv}}}


def moe(experts=4, top=2, ff=24):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top}}


def make_config(layers, width=64, vocab=48, max_positions=160, eps=1e-5,
                embed_scale=2.0):
    return {"architecture": "Gurapel", "embedding": {"scale": embed_scale},
            "layers": layers, "max_positions": max_positions,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_weights(cfg, seed=0, slow_decay=False):
    """bf16-representable random tensors under the checkpoint's names.
    slow_decay keeps the recurrent states' memory long (decays near 1) so
    that far-away tokens still matter."""
    gen = torch.Generator().manual_seed(seed)
    W = {}

    def rnd(name, *shape, std=1.0, mean=0.0):
        t = torch.randn(*shape, generator=gen) * std + mean
        W[name] = t.to(torch.bfloat16)

    width = cfg["width"]
    rnd("embed", cfg["vocab"], width)
    rnd("pos", cfg["max_positions"], width, std=0.5)
    rnd("final.norm", width, std=0.2)
    rnd("head", cfg["vocab"], width, std=width ** -0.5)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        rnd(p + "norm1", width, std=0.2)
        if L["type"] == "delta":
            m = L["mixer"]
            nqk, nv = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            q = p + "mix."
            for n, rows in (("q", nqk), ("k", nqk), ("v", nv)):
                rnd(q + n, rows, width, std=width ** -0.5)
                rnd(q + n + ".conv", rows, m["conv"], std=0.6)
            rnd(q + "b", m["heads"], width, std=width ** -0.5)
            rnd(q + "a", m["heads"], width, std=width ** -0.5)
            rnd(q + "A_log", m["heads"], std=0.5,
                mean=-4.0 if slow_decay else -0.5)
            rnd(q + "dt_bias", m["heads"], std=0.5)
            rnd(q + "norm", m["vdim"], std=0.3, mean=1.0)
            rnd(q + "g", nv, width, std=width ** -0.5)
            rnd(q + "o", width, nv, std=nv ** -0.5)
        else:
            a, r = L["mixer"]["left"], L["mixer"]["right"]
            q = p + "mix.left."
            rnd(q + "q", a["heads"] * a["dim"], width, std=width ** -0.5)
            rnd(q + "k", a["kv_heads"] * a["dim"], width, std=width ** -0.5)
            rnd(q + "v", a["kv_heads"] * a["vdim"], width, std=width ** -0.5)
            rnd(q + "q.norm", a["dim"], std=0.3, mean=1.0)
            rnd(q + "k.norm", a["dim"], std=0.3, mean=1.0)
            W[q + "r1"] = (torch.rand(a["heads"], generator=gen)
                           ).to(torch.bfloat16)
            W[q + "r2"] = (torch.rand(a["heads"], generator=gen) * 2
                           ).to(torch.bfloat16)
            rnd(q + "o", width, a["heads"] * a["vdim"],
                std=(a["heads"] * a["vdim"]) ** -0.5)
            q = p + "mix.right."
            w, nb = r["width"], r["blocks"]
            bw = w // nb
            rnd(q + "y", w, width, std=width ** -0.5)
            rnd(q + "y.b", w, std=0.2)
            rnd(q + "x", w, width, std=width ** -0.5)
            rnd(q + "x.b", w, std=0.2)
            rnd(q + "conv", w, r["conv"], std=0.6)
            rnd(q + "conv.b", w, std=0.2)
            rnd(q + "ra", nb, bw, bw, std=bw ** -0.5)
            rnd(q + "ra.b", nb, bw, std=0.3)
            rnd(q + "ri", nb, bw, bw, std=bw ** -0.5)
            rnd(q + "ri.b", nb, bw, std=0.3)
            rnd(q + "lam", w, std=0.5, mean=-5.0 if slow_decay else -1.0)
            rnd(q + "o", width, w, std=w ** -0.5)
            rnd(p + "mix.left.out", width, std=0.3, mean=1.0)
            rnd(p + "mix.right.out", width, std=0.3, mean=1.0)
        if L.get("mlp") is not None:
            m = L["mlp"]
            q = p + "mlp."
            rnd(p + "norm2", width, std=0.2)
            rnd(q + "router", m["router"]["experts"], width, std=0.5)
            ff = m["expert"]["ff"]
            for e in range(m["router"]["experts"]):
                rnd(f"{q}e{e}.gate", ff, width, std=width ** -0.5)
                rnd(f"{q}e{e}.up", ff, width, std=width ** -0.5)
                rnd(f"{q}e{e}.down", width, ff, std=ff ** -0.5)
    return W


def write_checkpoint(folder, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()},
              os.path.join(folder, "model.safetensors"))
    return folder
