"""Each sequence-mixer op of the hybrid stacks alone (kaito_amd.ops, CPU
reference and — under `-m gpu` — the HIP kernels, f32 and bf16) against the
plain functions of tests/hybrid_oracle.py, with inputs built so that a
window that is one key off, a lost tail or state, or a stale slot shows."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import hybrid_oracle as O  # noqa: E402

from kaito_amd import ops  # noqa: E402

MODES = [("cpu", torch.float32),
         pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu),
         pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)]
BS = 16   # page size


def close(got, want, dtype, scale=None):
    got, want = got.double().cpu(), want.double()
    lim = 3e-5 if dtype == torch.float32 else 2.5e-2
    ref = want.abs().max().item() if scale is None else scale
    assert (got - want).abs().max().item() <= lim * max(ref, 1e-6), \
        (got - want).abs().max().item() / max(ref, 1e-6)


def layout(dev, lens, starts, slots):
    cu, seq = [0], []
    for i, n in enumerate(lens):
        cu.append(cu[-1] + n)
        seq += [i] * n
    pos = [p for n, s in zip(lens, starts) for p in range(s, s + n)]
    t = lambda v, dt=torch.int32: torch.tensor(v, dtype=dt, device=dev)
    return t(cu), t(slots), t(starts), t(seq), t(pos, torch.long)


def split_runs(total, cuts):
    """[(start, length)] portions of a sequence of `total` tokens."""
    edges = [0] + list(cuts) + [total]
    return [(a, b - a) for a, b in zip(edges, edges[1:]) if b > a]


# ------------------------------------------------------------ convolution

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("taps,cuts", [(4, [1, 2, 3, 9, 10, 12]), (2, [5]),
                                       (3, [2, 4]), (1, [3]),
                                       (5, list(range(1, 14)))])
@pytest.mark.parametrize("C", [37, 64])
def test_short_conv_portions(mode, taps, cuts, C):
    dev, dt = mode
    T = 14
    x = torch.randn(T, C).to(dt)
    w, b = torch.randn(C, taps), torch.randn(C)
    want = O.silu(O.short_conv(x.double(), w.double(), b.double()))
    # slot 1 holds garbage from an earlier owner: a fresh sequence must
    # not see it
    state = torch.full((3, max(taps - 1, 1), C), 7.0).to(dt).to(dev)
    outs = []
    for start, n in split_runs(T, cuts):
        cu, sl, st, ts, _ = layout(dev, [n], [start], [1])
        outs.append(ops.causal_conv_update(
            x[start:start + n].to(dev), w.to(dev), b.to(dev), state, cu, sl,
            st, ts, act=1))
    close(torch.cat(outs), want, dt)


# -------------------------------------------------------------- delta rule

def plain_delta(q, k, v, gate, a, b, a_log, dt_bias, norm_w, eps):
    T, G, D = q.shape
    H, V = v.shape[1], v.shape[2]
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) / D ** 0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    out = torch.zeros(T, H, V, dtype=O.F64)
    for h in range(H):
        g = h // (H // G)
        S = torch.zeros(D, V, dtype=O.F64)
        for t in range(T):
            S = S * torch.exp(-torch.exp(a_log[h]) * torch.log1p(
                torch.exp(a[t, h] + dt_bias[h])))
            u = torch.sigmoid(b[t, h]) * (v[t, h] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, h] = S.T @ q[t, g]
    return (O.unit_rms(out, eps) * norm_w * O.silu(gate)).reshape(T, H * V)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("G,H,D,V", [(1, 2, 16, 24), (3, 3, 8, 8),
                                     (2, 4, 48, 40), (1, 1, 128, 64),
                                     (1, 2, 64, 130), (1, 2, 10, 12),
                                     (1, 1, 256, 20)])
@pytest.mark.parametrize("rows_per_lane", ["16", "32"])
def test_delta_rule_portions(mode, G, H, D, V, rows_per_lane, monkeypatch):
    # both register tilings of the single-wave kernel (the launcher picks by
    # the number of waves otherwise)
    monkeypatch.setenv("KAITO_DELTA_ROWS_PER_LANE", rows_per_lane)
    dev, dt = mode
    if dev == "cpu" and rows_per_lane == "32":
        pytest.skip("kernel tiling is a GPU matter")
    T = 29
    r = lambda *s: torch.randn(*s).to(dt)
    q, k, v, gate = r(T, G, D), r(T, G, D), r(T, H, V), r(T, H, V)
    a, b = r(T, H), r(T, H)
    a_log = torch.randn(H) * 0.5 - 2.0       # slow decay: old tokens count
    dt_bias, norm_w = torch.randn(H), torch.randn(V)
    want = plain_delta(*(t.double() for t in (q, k, v, gate, a, b, a_log,
                                              dt_bias, norm_w)), 1e-5)
    state = torch.full((2, H, D, V), 3.0, device=dev)   # stale content
    outs = []
    for start, n in split_runs(T, [1, 3, 11, 12, 20]):
        cu, sl, st, _, _ = layout(dev, [n], [start], [1])
        s = slice(start, start + n)
        outs.append(ops.gated_delta_rule(
            q[s].to(dev), k[s].to(dev), v[s].to(dev), gate[s].to(dev),
            a[s].to(dev), b[s].to(dev), a_log.to(dev), dt_bias.to(dev),
            norm_w.to(dev), state, cu, sl, st, 1e-6, 1e-5))
    close(torch.cat(outs), want, dt)
    assert torch.all(state[0] == 3.0)        # the other slot is untouched


# ------------------------------------------------------------------ RG-LRU

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("W,NB", [(48, 3), (30, 1), (160, 2)])
def test_rglru_portions_and_batch(mode, W, NB):
    dev, dt = mode
    bw = W // NB
    lens = [23, 6]
    seqs = []
    for n in lens:
        u, y = torch.randn(n, W).to(dt), torch.randn(n, W).to(dt)
        gates = torch.randn(NB, n, 2 * bw)
        seqs.append((u, y, gates))
    rate = torch.rand(W) * 0.3               # slow decay
    want = []
    for u, y, gates in seqs:
        g = gates.double().permute(1, 0, 2)
        rg = torch.sigmoid(g[..., :bw]).reshape(-1, W)
        ig = torch.sigmoid(g[..., bw:]).reshape(-1, W)
        aa = torch.exp(-rg * rate.double())
        S = torch.zeros(W, dtype=O.F64)
        rows = []
        for t in range(u.shape[0]):
            S = aa[t] * S + torch.sqrt(1 - aa[t] ** 2) * ig[t] * u[t].double()
            rows.append(S * O.gelu_tanh(y[t].double()))
        want.append(torch.stack(rows))
    state = torch.full((4, W), -5.0, device=dev)
    # both sequences advance together, in unequal portions
    got = [[], []]
    plan = [[(0, 0, 1), (1, 0, 2)], [(0, 1, 15)], [(0, 16, 7), (1, 2, 4)]]
    for step in plan:
        cu, sl, st, _, _ = layout(dev, [n for _, _, n in step],
                                  [s for _, s, _ in step],
                                  [3 if i == 0 else 0 for i, _, _ in step])
        u = torch.cat([seqs[i][0][s:s + n] for i, s, n in step]).to(dev)
        y = torch.cat([seqs[i][1][s:s + n] for i, s, n in step]).to(dev)
        gates = torch.cat([seqs[i][2][:, s:s + n] for i, s, n in step],
                          1).contiguous().to(dev)
        out = ops.rglru_scan(u, gates, y, rate.to(dev), state, cu, sl, st)
        at = 0
        for i, _, n in step:
            got[i].append(out[at:at + n])
            at += n
    for g, w in zip(got, want):
        close(torch.cat(g), w, dt)


@pytest.mark.parametrize("mode", MODES)
def test_rglru_prompt_sized_step(mode):
    """A step of long portions (the segment-parallel scan on the GPU):
    chunk borders inside segments, a carried state, a one-token chunk and
    a padding chunk."""
    dev, dt = mode
    W, NB = 96, 2
    bw = W // NB
    lens, starts, slots = [150, 1, 70, 9, 130], [0, 5, 33, 0, 64], \
        [2, 0, 1, -1, 3]
    T = sum(lens)
    u, y = torch.randn(T, W).to(dt), torch.randn(T, W).to(dt)
    gates = torch.randn(NB, T, 2 * bw)
    rate = torch.rand(W) * 0.2
    init = torch.randn(4, W)
    state = init.clone().to(dev)
    cu, sl, st, ts, _ = layout(dev, lens, starts, slots)
    got = ops.rglru_scan(u.to(dev), gates.to(dev), y.to(dev), rate.to(dev),
                         state, cu, sl, st, ts)
    g = gates.double().permute(1, 0, 2)
    rg = torch.sigmoid(g[..., :bw]).reshape(T, W)
    ig = torch.sigmoid(g[..., bw:]).reshape(T, W)
    aa = torch.exp(-rg * rate.double())
    at = 0
    for n, s0, slot in zip(lens, starts, slots):
        if slot >= 0:
            S = init[slot].double() if s0 > 0 else torch.zeros(W,
                                                               dtype=O.F64)
            rows = []
            for t in range(at, at + n):
                S = aa[t] * S + torch.sqrt(1 - aa[t] ** 2) * ig[t] \
                    * u[t].double()
                rows.append(S * O.gelu_tanh(y[t].double()))
            close(got[at:at + n], torch.stack(rows), dt)
            close(state[slot], S, torch.float32)
        at += n


# --------------------------------------------------------------- attention

def paged(dev, dt, G, D, V, n_pages=12):
    return (torch.zeros(n_pages, G, BS, D, dtype=dt, device=dev),
            torch.zeros(n_pages, G, BS, V, dtype=dt, device=dev))


def run_attention(dev, dt, q, k, v, runs, window, scale, cap, r1, r2,
                  qw=None, kw=None, eps=1e-5):
    """Feed one sequence through qk_norm_cache_write + window_attention in
    the given portions, pages deliberately out of order."""
    T, H, D = q.shape
    G, V = k.shape[1], v.shape[2]
    kc, vc = paged(dev, dt, G, D, V)
    pages = [7, 2, 9, 0, 5, 11, 3][:-(-T // BS)]
    bt = torch.tensor([pages + [0] * (8 - len(pages))], dtype=torch.int32,
                      device=dev)
    outs = []
    for start, n in runs:
        _, _, _, ts, pos = layout(dev, [n], [start], [0])
        slots = torch.tensor([pages[p // BS] * BS + p % BS
                              for p in range(start, start + n)],
                             dtype=torch.long, device=dev)
        s = slice(start, start + n)
        qn = ops.qk_norm_cache_write(
            q[s].to(dev), k[s].to(dev), v[s].to(dev),
            None if qw is None else qw.to(dev),
            None if kw is None else kw.to(dev), eps, kc, vc, slots)
        outs.append(ops.window_attention(
            qn, kc, vc, bt, ts, pos, scale, cap,
            None if r1 is None else r1.to(dev),
            None if r2 is None else r2.to(dev), window))
    return torch.cat(outs)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("H,G,D,V,window", [(4, 2, 16, 8, 11),
                                            (2, 1, 24, 40, 1),
                                            (3, 3, 8, 24, 21),
                                            (2, 2, 64, 128, 40),
                                            (2, 1, 16, 16, 0),
                                            (2, 1, 10, 12, 5),
                                            (16, 1, 16, 8, 9),
                                            (1, 1, 16, 320, 4)])
def test_window_attention_matches_plain(mode, H, G, D, V, window):
    dev, dt = mode
    T = 45
    r = lambda *s: torch.randn(*s).to(dt)
    q, k, v = r(T, H, D), r(T, G, D), r(T, G, V)
    qw, kw = torch.randn(D), torch.randn(D)
    r1, r2 = torch.rand(H), torch.rand(H) * 2
    qn = O.unit_rms(q.double(), 1e-5) * qw.double()
    kn = O.unit_rms(k.double(), 1e-5) * kw.double()
    want = O.window_attention(qn, kn, v.double(), window or T, 0.4, 3.0,
                              r1.double(), r2.double())
    for runs in ([(0, T)], split_runs(T, [1, 3, 15, 16, 17, 33]),
                 [(i, 1) for i in range(T)]):
        got = run_attention(dev, dt, q, k, v, runs, window, 0.4, 3.0, r1, r2,
                            qw, kw)
        close(got, want, dt)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("window", [5, 16, 17, 33])
@pytest.mark.parametrize("decode", [False, True])
def test_window_edge_stands_out(mode, window, decode):
    """One key gets a score far above all others; its value is a marker.
    The query `window - 1` tokens later must return the marker, the next
    query must not — in a prompt portion and decoded alone, with the key at,
    before and after page borders."""
    dev, dt = mode
    D, V, T = 8, 4, 60
    for key_pos in (0, 14, 15, 16, 26):
        q = torch.zeros(T, 1, D)
        k = torch.zeros(T, 1, D)
        v = torch.zeros(T, 1, V)
        k[:, 0, 1] = 1.0                       # every key: mild, equal
        k[key_pos, 0, 0] = 30.0                # the marked key
        v[key_pos, 0, 3] = 1.0
        q[:, 0, 0] = 30.0
        last_in = key_pos + window - 1
        if last_in + 1 >= T:
            continue
        runs = [(0, key_pos + 1)] + \
            ([(i, 1) for i in range(key_pos + 1, T)] if decode
             else [(key_pos + 1, T - key_pos - 1)])
        got = run_attention(dev, dt, q.to(dt), k.to(dt), v.to(dt), runs,
                            window, 1.0, 0.0, None, None).float().cpu()
        assert got[last_in, 0, 3] > 0.99       # just inside
        assert got[last_in + 1, 0, 3] < 1e-3   # just outside
        assert got[key_pos, 0, 3] > 0.99       # sees itself


@pytest.mark.parametrize("mode", MODES)
def test_distance_penalty_and_cap(mode):
    """Equal raw scores: the weights must follow (1 + r2 d)^-r1 exactly;
    huge raw scores: the cap bounds them."""
    dev, dt = mode
    T, D = 20, 8
    q = torch.zeros(T, 1, D)
    k = torch.zeros(T, 1, D)
    v = torch.zeros(T, 1, T)
    v[torch.arange(T), 0, torch.arange(T)] = 1.0   # output = the weights
    r1, r2 = torch.tensor([1.5]), torch.tensor([0.5])
    got = run_attention(dev, dt, q.to(dt), k.to(dt), v.to(dt), [(0, T)], 0,
                        1.0, 0.0, r1, r2).float().cpu()[T - 1, 0]
    d = torch.arange(T - 1, -1, -1, dtype=torch.float64)
    want = (1 + 0.5 * d) ** -1.5
    close(got, want / want.sum(), dt)
    q[:, 0, 0] = 100.0
    k[5, 0, 0] = 100.0
    k[9, 0, 0] = -100.0
    got = run_attention(dev, dt, q.to(dt), k.to(dt), v.to(dt), [(0, T)], 0,
                        1.0, 2.0, None, None).float().cpu()[T - 1, 0]
    s = torch.zeros(T, dtype=torch.float64)
    s[5], s[9] = 2.0, -2.0                     # tanh saturates at the cap
    close(got, torch.softmax(s, 0), dt)


# -------------------------------------------------------------------- norms

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("width", [64, 100, 1536])
def test_post_norm_residual(mode, width):
    dev, dt = mode
    T = 5
    x = torch.randn(T, width)
    y, y2 = torch.randn(T, width).to(dt), torch.randn(T, width).to(dt)
    w, wa, wb = torch.randn(width), torch.randn(width), torch.randn(width)
    x1 = x.clone().to(dev)
    xa = ops.post_norm_residual(x1, y.to(dev), w.to(dev), 1e-5, dt)
    want = x.double() + O.unit_rms(y.double(), 1e-5) * w.double()
    close(x1, want, torch.float32)
    close(xa, want, dt)
    m = 0.5 * (O.unit_rms(y.double(), 1e-5) * wa.double()
               + O.unit_rms(y2.double(), 1e-5) * wb.double())
    want2 = want + O.unit_rms(m, 1e-5) * w.double()
    ops.post_norm_residual(x1, y.to(dev), w.to(dev), 1e-5, dt,
                           y2=y2.to(dev), w_y=wa.to(dev), w_y2=wb.to(dev))
    close(x1, want2, torch.float32)
    close(ops.rms_norm_cast(x1, w.to(dev), 1e-5, dt),
          O.unit_rms(want2, 1e-5) * w.double(), dt)


# ---------------------------------------------------------------------- MoE

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("experts,top,ff,width", [(4, 2, 24, 64),
                                                  (3, 1, 40, 96),
                                                  (6, 3, 64, 128)])
def test_moe_router_and_experts(mode, experts, top, ff, width):
    """The engine's MoE layer configured as the hybrid stacks use it (f32
    router, softmax over the chosen logits, zero-padded expert width)."""
    import dataclasses
    from kaito_amd.engine.config import ModelConfig
    from kaito_amd.models.hybrid_config import MoESpec, layer_moe_config
    from kaito_amd.models.moe import MoEMLP
    from kaito_amd.parallel.state import init_parallel
    dev, dt = mode
    init_parallel(1)
    base = dataclasses.replace(ModelConfig(), hidden_size=width, dtype=dt)
    mlp = MoEMLP(layer_moe_config(base, MoESpec(experts, top, ff))).to(dev)
    cfg = O.make_config([O.delta_layer(mlp=O.moe(experts, top, ff))],
                        width=width)
    W = {k[len("l0.mlp."):]: v for k, v in O.random_weights(cfg, 3).items()
         if k.startswith("l0.mlp.")}
    ie = mlp.ie_local
    with torch.no_grad():
        mlp.gate.copy_(W["router"].float())
        mlp.w_gate_up.zero_()
        mlp.w_down.zero_()
        for e in range(experts):
            mlp.w_gate_up[e, :ff].copy_(W[f"e{e}.gate"])
            mlp.w_gate_up[e, ie:ie + ff].copy_(W[f"e{e}.up"])
            mlp.w_down[e, :, :ff].copy_(W[f"e{e}.down"])
    x = torch.randn(9, width).to(dt)
    want = O.moe_ff(x.double(), {"p." + k: v.double() for k, v in W.items()},
                    "p.", cfg["layers"][0]["mlp"])
    close(mlp(x.to(dev)), want, dt)


# ------------------------------------------- MFMA prompt-portion attention

@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V,window", [(4, 1, 64, 128, 96),
                                            (2, 2, 128, 64, 70),
                                            (2, 1, 64, 64, 0),
                                            (4, 2, 128, 128, 33),
                                            (1, 1, 256, 256, 130)])
def test_window_attention_tiled_prompt_kernel(H, G, D, V, window):
    """Several chunks of one step (fresh prompts, continued portions that
    start inside a page and inside a window, a single token) on the tiled
    MFMA kernel against the plain attention."""
    dev, dt = "cuda", torch.bfloat16
    # (start, length): history before `start` is fed by an earlier step
    chunks = [(0, 150), (37, 70), (200, 1), (5, 64), (130, 3)]
    r1, r2 = torch.rand(H), torch.rand(H) * 2
    n_pages = sum(-(-(s + n) // BS) for s, n in chunks) + 1
    kc, vc = paged(dev, dt, G, D, V, n_pages)
    free = list(range(n_pages))[::-1]
    seqs, tables = [], []
    for s, n in chunks:
        T = s + n
        q = torch.randn(T, H, D).to(dt)
        k = torch.randn(T, G, D).to(dt)
        v = torch.randn(T, G, V).to(dt)
        pages = [free.pop() for _ in range(-(-T // BS))]
        seqs.append((q, k, v, pages))
        tables.append(pages)
    mb = max(len(p) for p in tables)
    bt = torch.tensor([p + [0] * (mb - len(p)) for p in tables],
                      dtype=torch.int32, device=dev)

    def slots(pages, a, b):
        return torch.tensor([pages[p // BS] * BS + p % BS
                             for p in range(a, b)], dtype=torch.long,
                            device=dev)

    # step 1: histories, each sequence alone (no norm weights: plain write)
    for (s, n), (q, k, v, pages) in zip(chunks, seqs):
        if s:
            ops.qk_norm_cache_write(q[:s].to(dev), k[:s].to(dev),
                                    v[:s].to(dev), None, None, 1e-5, kc, vc,
                                    slots(pages, 0, s))
    # step 2: all chunks together
    cu, sl, st, ts, pos = layout(dev, [n for _, n in chunks],
                                 [s for s, _ in chunks],
                                 list(range(len(chunks))))
    qs = torch.cat([q[s:s + n] for (s, n), (q, _, _, _) in zip(chunks, seqs)])
    ks = torch.cat([k[s:s + n] for (s, n), (_, k, _, _) in zip(chunks, seqs)])
    vs = torch.cat([v[s:s + n] for (s, n), (_, _, v, _) in zip(chunks, seqs)])
    sm = torch.cat([slots(p, s, s + n)
                    for (s, n), (_, _, _, p) in zip(chunks, seqs)])
    qn = ops.qk_norm_cache_write(qs.to(dev), ks.to(dev), vs.to(dev), None,
                                 None, 1e-5, kc, vc, sm)
    tiles = ops.build_query_tiles([n for _, n in chunks], dev) + (cu, st)
    got = ops.window_attention(qn, kc, vc, bt, ts, pos, 0.1, 4.0,
                               r1.to(dev), r2.to(dev), window, tiles=tiles)
    plain = ops.window_attention(qn, kc, vc, bt, ts, pos, 0.1, 4.0,
                                 r1.to(dev), r2.to(dev), window)
    at = 0
    for (s, n), (q, k, v, _) in zip(chunks, seqs):
        want = O.window_attention(q.double(), k.double(), v.double(),
                                  window or s + n, 0.1, 4.0, r1.double(),
                                  r2.double())[s:]
        close(got[at:at + n], want, dt)
        close(plain[at:at + n], want, dt)
        at += n
