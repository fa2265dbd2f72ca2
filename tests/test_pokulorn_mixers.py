"""Each mechanism of the Pokulorn stack alone (kaito_amd.ops, CPU reference
and — under `-m gpu` — the HIP kernels, f32 and bf16) against the plain
functions of tests/pokulorn_oracle.py, with inputs built so that a window
or a kept-first-tokens border that is one key off, a left-out sink, a lost
state or a stale slot shows."""
import math
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import pokulorn_oracle as P  # noqa: E402

from kaito_amd import ops  # noqa: E402
from kaito_amd.models.hybrid_config import RotarySpec  # noqa: E402

MODES = [("cpu", torch.float32),
         pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu),
         pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)]
BS = 16   # page size


def close(got, want, dtype, scale=None, slack=1.0):
    got = got.double().cpu()
    want = torch.as_tensor(np.asarray(want), dtype=torch.float64)
    lim = (3e-5 if dtype == torch.float32 else 2.5e-2) * slack
    ref = want.abs().max().item() if scale is None else scale
    err = (got - want).abs().max().item() / max(ref, 1e-6)
    assert err <= lim, err


def layout(dev, lens, starts, slots):
    cu, seq = [0], []
    for i, n in enumerate(lens):
        cu.append(cu[-1] + n)
        seq += [i] * n
    pos = [p for n, s in zip(lens, starts) for p in range(s, s + n)]
    t = lambda v, dt=torch.int32: torch.tensor(v, dtype=dt, device=dev)  # noqa: E731
    return t(cu), t(slots), t(starts), t(seq), t(pos, torch.long)


def split_runs(total, cuts):
    edges = [0] + list(cuts) + [total]
    return [(a, b - a) for a, b in zip(edges, edges[1:]) if b > a]


def f64(t):
    return t.double().numpy()


# ---------------------------------------------------------------- rotation

@pytest.mark.parametrize("rot", [
    P.rot(16), P.rot(8, base=500.0),
    P.rot(32, base=40000.0, scaling=(4.0, 64, 32.0, 1.0)),
    P.rot(16, base=10000.0, scaling=(2.0, 4096, 16.0, 2.0)),
    P.rot(64, base=1e6, scaling=(16.0, 128, 32.0, 1.0))])
def test_rotary_frequencies(rot):
    sc = rot.get("scaling") or {}
    spec = RotarySpec(dims=rot["dims"], base=rot["base"],
                      factor=sc.get("factor", 0.0),
                      original=sc.get("original", 0.0),
                      fast=sc.get("fast", 32.0), slow=sc.get("slow", 1.0))
    freq, mag = spec.frequencies()
    pos = [0, 1, 7, 300]
    cos, sin = P.rotary_tables(rot, pos)
    ang = np.outer(pos, freq)
    assert np.allclose(np.cos(ang) * mag, cos, atol=1e-12)
    assert np.allclose(np.sin(ang) * mag, sin, atol=1e-12)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("H,G,D,V,dims", [(4, 2, 16, 8, 16), (3, 1, 24, 20, 8),
                                          (2, 2, 64, 32, 32), (1, 1, 10, 6, 4)])
def test_norm_rotation_blend_cache_write(mode, H, G, D, V, dims):
    """q/k: per-head RMS norm then rotation of the first `dims` dims at the
    rows' own positions (far along the sequence too); v: blended with
    another layer's values; k and v land in the right page rows."""
    dev, dt = mode
    T = 9
    rot = P.rot(dims, base=3000.0, scaling=(3.0, 32, 8.0, 1.0))
    spec = RotarySpec(dims=dims, base=3000.0, factor=3.0, original=32,
                      fast=8.0, slow=1.0)
    freq, mag = spec.frequencies()
    inv_freq = torch.tensor(freq, dtype=torch.float64).float().to(dev)
    pos = [0, 1, 2, 15, 16, 17, 500, 4000, 4001]
    r = lambda *s: torch.randn(*s).to(dt)  # noqa: E731
    q, k, v, vf = r(T, H, D), r(T, G, D), r(T, G, V), r(T, G, V)
    qw, kw = torch.randn(D), torch.randn(D)
    lam = 0.3
    cos, sin = P.rotary_tables(rot, pos)
    want_q = P.rotate(P.rms(f64(q), 1e-5) * f64(qw), cos, sin)
    want_k = P.rotate(P.rms(f64(k), 1e-5) * f64(kw), cos, sin)
    want_v = (1 - lam) * f64(v) + lam * f64(vf)
    kc = torch.zeros(6, G, BS, D, dtype=dt, device=dev)
    vc = torch.zeros(6, G, BS, V, dtype=dt, device=dev)
    slots = torch.tensor([5 * BS + 15, 0, 2 * BS + 3, 17, 18, 3 * BS, 40, 41,
                          4 * BS + 9], dtype=torch.long, device=dev)
    qn = ops.qk_norm_cache_write(
        q.to(dev), k.to(dev), v.to(dev), qw.to(dev), kw.to(dev), 1e-5, kc, vc,
        slots, positions=torch.tensor(pos, dtype=torch.long, device=dev),
        inv_freq=inv_freq, rot_mag=mag, v_first=vf.to(dev), v_lambda=lam)
    # an angle of thousands of radians carries the f32 rounding of the
    # frequency: allow for it at the far positions
    close(qn, want_q, dt, slack=40)
    close(qn[:6], want_q[:6], dt)
    sl = slots.cpu()
    got_k = kc.cpu()[sl // BS, :, sl % BS]
    got_v = vc.cpu()[sl // BS, :, sl % BS]
    close(got_k[:6], want_k[:6], dt)
    close(got_k, want_k, dt, slack=40)
    close(got_v, want_v, dt)


# --------------------------------------------------------------- attention

def run_attention(dev, dt, q, k, v, runs, window, keep_first, scale, sinks,
                  tiled=False):
    """One sequence through qk_norm_cache_write (no norm, no rotation) +
    window_attention in the given portions, pages out of order."""
    T, H, D = q.shape
    G, V = k.shape[1], v.shape[2]
    kc = torch.zeros(12, G, BS, D, dtype=dt, device=dev)
    vc = torch.zeros(12, G, BS, V, dtype=dt, device=dev)
    pages = [7, 2, 9, 0, 5, 11, 3, 1][:-(-T // BS)]
    bt = torch.tensor([pages + [0] * (8 - len(pages))], dtype=torch.int32,
                      device=dev)
    outs = []
    for start, n in runs:
        cu, _, st, ts, pos = layout(dev, [n], [start], [0])
        slots = torch.tensor([pages[p // BS] * BS + p % BS
                              for p in range(start, start + n)],
                             dtype=torch.long, device=dev)
        s = slice(start, start + n)
        qn = ops.qk_norm_cache_write(q[s].to(dev), k[s].to(dev), v[s].to(dev),
                                     None, None, 1e-5, kc, vc, slots)
        tiles = None
        if tiled:
            tiles = ops.build_query_tiles([n], dev) + (cu, st)
        outs.append(ops.window_attention(
            qn, kc, vc, bt, ts, pos, scale, window=window, tiles=tiles,
            keep_first=keep_first,
            sinks=None if sinks is None else sinks.to(dev)))
    return torch.cat(outs)


def plain_attention(q, k, v, window, keep_first, scale, sinks):
    """Softmax over the visible keys, the sink only in the denominator."""
    T, H, D = q.shape
    G, V = k.shape[1], v.shape[2]
    out = np.zeros((T, H, V))
    for i in range(T):
        js = [j for j in range(i + 1)
              if window <= 0 or i - j < window or j < keep_first]
        for h in range(H):
            g = h // (H // G)
            s = np.array([q[i, h] @ k[j, g] for j in js]) * scale
            e = np.exp(s - s.max())
            den = e.sum() + (math.exp(sinks[h] - s.max())
                             if sinks is not None else 0.0)
            out[i, h] = (e / den) @ v[js, g]
    return out


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("H,G,D,V,window,keep,sink", [
    (4, 2, 16, 8, 11, 3, True), (2, 1, 24, 40, 1, 0, True),
    (3, 3, 8, 24, 21, 17, False), (2, 2, 64, 32, 20, 20, True),
    (2, 1, 16, 16, 0, 0, True), (2, 1, 10, 12, 5, 30, False),
    (16, 1, 16, 8, 9, 1, True), (1, 1, 16, 320, 4, 2, False)])
def test_attention_window_first_tokens_sink(mode, H, G, D, V, window, keep,
                                            sink):
    dev, dt = mode
    T = 50
    r = lambda *s: torch.randn(*s).to(dt)  # noqa: E731
    q, k, v = r(T, H, D), r(T, G, D), r(T, G, V)
    sinks = torch.randn(H) * 2 if sink else None
    want = plain_attention(f64(q), f64(k), f64(v), window, keep, 0.4,
                           None if sinks is None else f64(sinks))
    for runs in ([(0, T)], split_runs(T, [1, 3, 15, 16, 17, 33]),
                 [(i, 1) for i in range(T)]):
        got = run_attention(dev, dt, q, k, v, runs, window, keep, 0.4, sinks)
        close(got, want, dt)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("window,keep", [(5, 0), (16, 2), (17, 16), (33, 17),
                                         (8, 1)])
@pytest.mark.parametrize("decode", [False, True])
def test_window_and_first_token_edges_stand_out(mode, window, keep, decode):
    """One key gets a score far above all others; its value is a marker.
    A marked key beyond the kept first tokens is seen by the query
    `window - 1` tokens later and not by the next one; a marked key among
    the kept first tokens is seen to the end, the first key after them is
    not — in a prompt portion and decoded alone, keys at, before and after
    page borders."""
    dev, dt = mode
    D, V, T = 8, 4, 70
    for key_pos in (0, keep - 1, keep, 14, 15, 16, 26):
        if key_pos < 0:
            continue
        q = torch.zeros(T, 1, D)
        k = torch.zeros(T, 1, D)
        v = torch.zeros(T, 1, V)
        k[:, 0, 1] = 1.0                       # every key: mild, equal
        k[key_pos, 0, 0] = 30.0                # the marked key
        v[key_pos, 0, 3] = 1.0
        q[:, 0, 0] = 30.0
        runs = [(0, key_pos + 1)] + \
            ([(i, 1) for i in range(key_pos + 1, T)] if decode
             else [(key_pos + 1, T - key_pos - 1)])
        got = run_attention(dev, dt, q.to(dt), k.to(dt), v.to(dt), runs,
                            window, keep, 1.0, None).float().cpu()
        assert got[key_pos, 0, 3] > 0.99           # sees itself
        last_in = key_pos + window - 1
        if key_pos < keep:
            assert got[T - 1, 0, 3] > 0.99         # kept for good
            assert got[min(last_in + 1, T - 1), 0, 3] > 0.99
        elif last_in + 1 < T:
            assert got[last_in, 0, 3] > 0.99       # just inside
            assert got[last_in + 1, 0, 3] < 1e-3   # just outside


@pytest.mark.parametrize("mode", MODES)
def test_sink_counts_once_unscaled(mode):
    """All scores zero: n visible keys share 1 - e^s / (n + e^s) equally,
    whatever the score scale."""
    dev, dt = mode
    T, H = 12, 2
    q = torch.zeros(T, H, 8)
    k = torch.zeros(T, 1, 8)
    v = torch.ones(T, 1, 4)
    sinks = torch.tensor([math.log(3.0), -1.0])
    got = run_attention(dev, dt, q.to(dt), k.to(dt), v.to(dt), [(0, 5)] +
                        [(i, 1) for i in range(5, T)], 0, 0, 7.0,
                        sinks).float().cpu()
    for i in range(T):
        for h in range(H):
            e = math.exp(sinks[h].item())
            assert abs(got[i, h, 0].item() - (i + 1) / (i + 1 + e)) < \
                (1e-5 if dt == torch.float32 else 1e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V,window,keep,sink", [
    (4, 1, 64, 32, 48, 24, True), (2, 2, 64, 64, 0, 0, False),
    (2, 1, 128, 32, 70, 33, True), (2, 2, 64, 128, 33, 64, False),
    (2, 1, 64, 32, 100, 5, True)])
def test_tiled_prompt_kernel_window_first_tokens_sink(H, G, D, V, window,
                                                      keep, sink):
    """The MFMA prompt kernel (bf16) against the plain attention: portions
    that start inside tiles, key tiles skipped between the kept first
    tokens and the window."""
    dev, dt = "cuda", torch.bfloat16
    T = 128
    r = lambda *s: torch.randn(*s).to(dt)  # noqa: E731
    q, k, v = r(T, H, D), r(T, G, D), r(T, G, V)
    sinks = torch.randn(H) * 2 if sink else None
    want = plain_attention(f64(q), f64(k), f64(v), window, keep, 0.2,
                           None if sinks is None else f64(sinks))
    for runs in ([(0, T)], split_runs(T, [9, 70, 71, 100])):
        got = run_attention(dev, dt, q, k, v, runs, window, keep, 0.2, sinks,
                            tiled=True)
        close(got, want, dt)


# ------------------------------------------------------------ matrix memory

def plain_mlstm(q, k, v, gate, ipre, fpre, norm_w, cap, eps):
    T, H, D = q.shape
    V = v.shape[2]
    gi = cap * np.tanh(ipre / cap)
    gf = P.log_sigmoid(cap * np.tanh(fpre / cap))
    o = np.zeros((T, H, V))
    for h in range(H):
        C, n, m = np.zeros((D, V)), np.zeros(D), 0.0
        for t in range(T):
            m2 = max(gf[t, h] + m, gi[t, h])
            a, b = math.exp(gf[t, h] + m - m2), math.exp(gi[t, h] - m2)
            C = a * C + b * np.outer(k[t, h], v[t, h])
            n = a * n + b * k[t, h]
            m = m2
            qs = q[t, h] * D ** -0.5
            o[t, h] = C.T @ qs / (max(abs(n @ qs), math.exp(-m)) + 1e-6)
    o = P.rms(o, eps).reshape(T, H * V) * norm_w
    return o * P.sigmoid(gate.reshape(T, H * V))


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("H,D,V,cap", [(2, 16, 24, 15.0), (3, 8, 8, 4.0),
                                       (1, 56, 40, 11.0), (2, 10, 17, 8.0),
                                       (1, 128, 64, 20.0), (4, 24, 15, 2.0)])
def test_mlstm_portions_and_stale_slots(mode, H, D, V, cap):
    dev, dt = mode
    T = 31
    r = lambda *s: torch.randn(*s).to(dt)  # noqa: E731
    q, k, v, gate = r(T, H, D), r(T, H, D), r(T, H, V), r(T, H, V)
    # gate pre-activations wide enough that the cap and the running
    # maximum both matter; forget gates mostly open so old tokens count
    ipre = torch.randn(T, H) * cap
    fpre = torch.randn(T, H) * 3 + 4
    norm_w = torch.randn(H * V)
    want = plain_mlstm(f64(q), f64(k), f64(v), f64(gate), f64(ipre),
                       f64(fpre), f64(norm_w), cap, 1e-5)
    # slot 1 holds another sequence's leftovers
    sc = torch.full((2, H, D, V), 3.0, device=dev)
    sn = torch.full((2, H, D), -2.0, device=dev)
    sm = torch.full((2, H), 5.0, device=dev)
    outs = []
    for start, n in split_runs(T, [1, 3, 11, 12, 20]):
        cu, sl, st, _, _ = layout(dev, [n], [start], [1])
        s = slice(start, start + n)
        outs.append(ops.mlstm_scan(
            q[s].to(dev), k[s].to(dev), v[s].to(dev), gate[s].to(dev),
            ipre[s].to(dev), fpre[s].to(dev), norm_w.to(dev), sc, sn, sm, cu,
            sl, st, cap, D ** -0.5, 1e-5))
    close(torch.cat(outs), want, dt, slack=2)
    assert torch.all(sc[0] == 3.0) and torch.all(sm[0] == 5.0)


@pytest.mark.parametrize("mode", MODES)
def test_mlstm_long_chunks_beside_short(mode):
    """Chunks of several hundred tokens (the running maximum is scanned in
    parallel runs inside a chunk) beside a single-token chunk; input gates
    that jump so that the maximum is reset in the middle of runs."""
    dev, dt = mode
    H, D, V, cap = 2, 8, 12, 10.0
    lens = [333, 1, 130]
    r = lambda *s: torch.randn(*s).to(dt)  # noqa: E731
    norm_w = torch.randn(H * V)
    seqs, want = [], []
    for n in lens:
        ipre = torch.randn(n, H) * 4
        ipre[torch.rand(n, H) < 0.03] += 25.0
        s = (r(n, H, D), r(n, H, D), r(n, H, V), r(n, H, V), ipre,
             torch.randn(n, H) * 2 + 3)
        seqs.append(s)
        want.append(plain_mlstm(*(f64(t) for t in s), f64(norm_w), cap,
                                1e-5))
    sc = torch.full((3, H, D, V), 1.0, device=dev)
    sn = torch.full((3, H, D), 1.0, device=dev)
    sm = torch.full((3, H), -3.0, device=dev)
    got = [[] for _ in lens]
    for cut in ((0, 200), (200, 400)):
        parts_in, lens_now, starts, slots, owner = [], [], [], [], []
        for i, n in enumerate(lens):
            a, b = min(cut[0], n), min(cut[1], n)
            if b > a:
                parts_in.append([t[a:b] for t in seqs[i]])
                lens_now.append(b - a)
                starts.append(a)
                slots.append(i)
                owner.append(i)
        cat = [torch.cat([p[j] for p in parts_in]).to(dev) for j in range(6)]
        cu, sl, st, _, _ = layout(dev, lens_now, starts, slots)
        out = ops.mlstm_scan(cat[0], cat[1], cat[2], cat[3], cat[4], cat[5],
                             norm_w.to(dev), sc, sn, sm, cu, sl, st, cap,
                             D ** -0.5, 1e-5)
        row = 0
        for i, n in zip(owner, lens_now):
            got[i].append(out[row:row + n])
            row += n
    for g, w in zip(got, want):
        close(torch.cat(g), w, dt, slack=3)


@pytest.mark.parametrize("mode", MODES)
def test_mlstm_running_maximum_starts_at_zero(mode):
    """Strongly negative input gates at the start: with the maximum
    starting at 0 (not at minus infinity) the first read-outs are divided
    by exp(-m) = 1, not renormalised to full size. The output gate is wide
    open and the norm is skipped by looking at ratios inside one head."""
    dev, dt = mode
    T, H, D, V = 4, 1, 8, 8
    q = torch.ones(T, H, D).to(dt)
    k = torch.ones(T, H, D).to(dt)
    v = torch.zeros(T, H, V)
    v[:, 0, 0] = 1.0
    v[:, 0, 1] = torch.tensor([1.0, 2.0, 3.0, 4.0])
    gate = torch.zeros(T, H, V).to(dt)
    ipre = torch.full((T, H), -6.0)
    fpre = torch.full((T, H), 8.0)
    want = plain_mlstm(f64(q), f64(k), f64(v), f64(gate), f64(ipre),
                       f64(fpre), np.ones(H * V), 30.0, 1e-6)
    cu, sl, st, _, _ = layout(dev, [T], [0], [0])
    sc = torch.zeros(1, H, D, V, device=dev)
    sn = torch.zeros(1, H, D, device=dev)
    sm = torch.zeros(1, H, device=dev)
    got = ops.mlstm_scan(q.to(dev), k.to(dev), v.to(dt).to(dev), gate.to(dev),
                         ipre.to(dev), fpre.to(dev), torch.ones(H * V,
                                                                device=dev),
                         sc, sn, sm, cu, sl, st, 30.0, D ** -0.5, 1e-6)
    close(got, want, dt)
    assert abs(sm.item()) < 1e-2            # max(f + m, -6) stays near 0


# --------------------------------------------------------------- state space

def plain_ssd(x, B, C, dt, z, a_log, dt_bias, d_skip, norm_w, parts, eps):
    T, H, Pd = x.shape
    G, N = B.shape[1], B.shape[2]
    step = P.softplus(dt + dt_bias)
    y = np.zeros((T, H, Pd))
    for h in range(H):
        g = h // (H // G)
        S = np.zeros((N, Pd))
        for t in range(T):
            S = math.exp(-math.exp(a_log[h]) * step[t, h]) * S \
                + step[t, h] * np.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + d_skip[h] * x[t, h]
    y = y.reshape(T, H * Pd) * P.silu(z)
    y = P.rms(y.reshape(T, parts, -1), eps).reshape(T, H * Pd)
    return y * norm_w


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("H,Pd,N,G,parts", [(4, 8, 16, 2, 2), (3, 20, 12, 3, 1),
                                            (6, 16, 24, 1, 3), (2, 64, 128, 2, 4),
                                            (1, 5, 7, 1, 1)])
def test_ssd_portions_batch_and_padding(mode, H, Pd, N, G, parts):
    """Two sequences advance in the same steps (one in portions, one token
    by token) beside a padding chunk; slots hold stale state."""
    dev, dt = mode
    lens = [27, 6]
    r = lambda *s: torch.randn(*s).to(dt)  # noqa: E731
    a_log = torch.randn(H) * 0.5 - 2.0          # slow decay
    dt_bias, d_skip = torch.randn(H), torch.randn(H)
    norm_w = torch.randn(H * Pd)
    seqs, want = [], []
    for n in lens:
        s = (r(n, H, Pd), r(n, G, N), r(n, G, N), torch.randn(n, H),
             r(n, H * Pd))
        seqs.append(s)
        want.append(plain_ssd(*(f64(t) for t in s), f64(a_log), f64(dt_bias),
                              f64(d_skip), f64(norm_w), parts, 1e-5))
    state = torch.full((4, H, N, Pd), 9.0, device=dev)
    got = [[], []]
    at = [0, 0]
    plan = [(5, 1), (2, 1), (9, 1), (1, 1), (10, 1), (0, 1)]
    for n0, n1 in plan:
        parts_in, lens_now, starts, slots, owner = [], [], [], [], []
        for i, n in ((0, n0), (1, n1)):
            n = min(n, lens[i] - at[i])
            if n <= 0:
                continue
            parts_in.append([t[at[i]:at[i] + n] for t in seqs[i]])
            lens_now.append(n)
            starts.append(at[i])
            slots.append(2 if i == 0 else 0)
            owner.append(i)
            at[i] += n
        # a padding chunk of one row between the live ones
        lens_now.insert(1, 1)
        starts.insert(1, 0)
        slots.insert(1, -1)
        pad = [t[:1] for t in seqs[0]]
        parts_in.insert(1, pad)
        owner.insert(1, None)
        cat = [torch.cat([p[j] for p in parts_in]).to(dev) for j in range(5)]
        cu, sl, st, _, _ = layout(dev, lens_now, starts, slots)
        out = ops.ssd_scan(cat[0], cat[1], cat[2], cat[3], cat[4],
                           a_log.to(dev), dt_bias.to(dev), d_skip.to(dev),
                           norm_w.to(dev), state, cu, sl, st, parts, 1e-5)
        row = 0
        for i, n in zip(owner, lens_now):
            if i is not None:
                got[i].append(out[row:row + n])
            row += n
    assert at == lens
    for g, w in zip(got, want):
        close(torch.cat(g), w, dt, slack=2)
    assert torch.all(state[1] == 9.0) and torch.all(state[3] == 9.0)


# ------------------------------------------------------- residual, gates

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("width", [64, 100, 1536])
def test_residual_add_norm(mode, width):
    dev, dt = mode
    T = 5
    x = torch.randn(T, width)
    y, y2 = torch.randn(T, width).to(dt), torch.randn(T, width).to(dt)
    w = torch.randn(width)
    x32 = x.clone().to(dev)
    h = ops.residual_add_norm(x32, y.to(dev), w.to(dev), 1e-5, dt)
    s = f64(x) + f64(y)
    close(x32, s, torch.float32)
    close(h, P.rms(s, 1e-5) * f64(w), dt)
    x32 = x.clone().to(dev)
    h = ops.residual_add_norm(x32, y.to(dev), w.to(dev), 1e-5, dt,
                              y2=y2.to(dev), s1=0.6, s2=-1.5)
    s = f64(x) + 0.6 * f64(y) - 1.5 * f64(y2)
    close(x32, s, torch.float32)
    close(h, P.rms(s, 1e-5) * f64(w), dt)
    x32 = x.clone().to(dev)
    assert ops.residual_add_norm(x32, y.to(dev), None, 1e-5, dt) is None
    close(x32, f64(x) + f64(y), torch.float32)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("ff,limit", [(24, 1.0), (130, 7.0)])
def test_clamped_glu_and_sigmoid_gate(mode, ff, limit):
    dev, dt = mode
    gu = (torch.randn(7, 2 * ff) * 3).to(dt)
    g = np.minimum(f64(gu)[:, :ff], limit)
    u = np.clip(f64(gu)[:, ff:], -limit, limit)
    close(ops.clamped_glu(gu.to(dev), limit, 1.702),
          g * P.sigmoid(1.702 * g) * (u + 1), dt)
    big = torch.randn(7, 3 * ff).to(dt)
    x, gate = big[:, :ff].contiguous(), big[:, ff:2 * ff]   # strided gate
    close(ops.sigmoid_mul(x.to(dev), gate.to(dev)),
          f64(x) * P.sigmoid(f64(gate)), dt)
