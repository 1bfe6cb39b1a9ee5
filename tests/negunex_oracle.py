"""Plain float64 implementation of the Negunex design, one function per mechanism, written from
its equations and sharing no code with llmd_amd. Slow on purpose: whole sequences, dense
attention matrices, Python loops over heads, tokens and experts.

A model is (cfg, w): ``cfg`` the design's config.json as a dict, ``w`` name -> tensor with the
checkpoint's names. ``forward(cfg, w, tokens)`` returns (logits [T, vocab], per-layer sums of the
streams [L, T, width]).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(var + eps) * weight, var = mean of squared deviations; no bias."""
    x = x.to(F64)
    mu = x.mean(-1, keepdim=True)
    dev = x - mu
    var = (dev * dev).mean(-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * weight.to(F64)


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis, no weight."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2; with ``scaling`` (factor, low, high, original) the
    long wavelengths are slowed down by ``factor``, the short ones kept, a linear blend between."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelen = 2.0 * math.pi / f
            if wavelen < orig / hi:
                pass
            elif wavelen > orig / lo:
                f = f / fac
            else:
                s = (orig / wavelen - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return out


def rotate_interleaved(x, positions, dims, base, scaling=None):
    """x [T, heads, dim]: dimensions (2i, 2i+1), i < dims/2, turn by positions * f_i; the rest pass."""
    x = x.clone()
    freqs = rotary_frequencies(dims, base, scaling)
    for t, p in enumerate(positions):
        for i, f in enumerate(freqs):
            a = float(p) * f
            c, s = math.cos(a), math.sin(a)
            u, v = x[t, :, 2 * i].clone(), x[t, :, 2 * i + 1].clone()
            x[t, :, 2 * i] = u * c - v * s
            x[t, :, 2 * i + 1] = v * c + u * s
    return x


def causal_softmax_attention(q, k, v, scale):
    """q [T, H, dim], k [T, G, dim], v [T, G, vdim]; query head h reads key/value head
    h // (H / G); token i sees j <= i. Returns [T, H, vdim]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(torch.ones(T, T).triu(1).bool(), float("-inf"))
        out[:, h] = torch.softmax(s, -1) @ v[:, g]
    return out


def attention_mixer(h, w, pre, m, eps, positions, v_first):
    """One attention mixer on input h [T, width]. ``v_first``: values of the first value-mixing
    layer (None in that layer itself or without value mixing). Returns (output, this layer's values
    before mixing)."""
    h = h.to(F64)
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    g = lambda n: w[pre + n].to(F64)  # noqa: E731
    q = (h @ g("q").T + g("q.b")).view(T, H, dim)
    k = (h @ g("k").T + g("k.b")).view(T, G, dim)
    v = (h @ g("v").T + g("v.b")).view(T, G, vdim)
    rot = m.get("rot")
    if rot:
        q = rotate_interleaved(q, positions, rot["dims"], rot["base"], rot.get("scaling"))
        k = rotate_interleaved(k, positions, rot["dims"], rot["base"], rot.get("scaling"))
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    v_own = v
    if m.get("v_mix") and v_first is not None:
        lam = g("vmix")
        v = (1.0 - lam) * v + lam * v_first
    o = causal_softmax_attention(q, k, v, float(m["scale"])).reshape(T, H * vdim)
    o = o * torch.sigmoid(h @ g("g").T)
    return o @ g("o").T, v_own


def dense_ff(h, w, pre):
    h = h.to(F64)
    g = lambda n: w[pre + n].to(F64)  # noqa: E731
    return (gelu_tanh(h @ g("gate").T) * (h @ g("up").T)) @ g("down").T


def route(h, router, correction, top):
    """Softmax over all router outputs; the ``top`` largest of (score + correction) are chosen;
    weights = their scores / (sum + 1e-20). Returns (ids [T, top], weights [T, top])."""
    s = torch.softmax(h.to(F64) @ router.to(F64).T, -1)
    ids = torch.topk(s + correction.to(F64), top, dim=-1).indices
    ws = torch.gather(s, 1, ids)
    return ids, ws / (ws.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, w, pre, mlp):
    h = h.to(F64)
    r = mlp["router"]
    E = r["experts"]
    ids, ws = route(h, w[pre + "router"], w[pre + "correction"], r["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            if e >= E:  # identity expert: the input itself
                y = h[t]
            else:
                g = lambda n: w[f"{pre}e{e}.{n}"].to(F64)  # noqa: E731
                y = g("down") @ (silu(g("gate") @ h[t]) * (g("up") @ h[t]))
            out[t] += ws[t, j] * y
    return out


def hyper_in(streams, w_in):
    """u = sum_s in[s] x_s."""
    return sum(w_in[s].to(F64) * streams[s] for s in range(len(streams)))


def hyper_out(streams, y, w_mix, w_out):
    """x_t <- sum_s mix[s, t] x_s + out[t] y, all from the old streams."""
    S = len(streams)
    return [sum(w_mix[s, t].to(F64) * streams[s] for s in range(S)) + w_out[t].to(F64) * y for t in range(S)]


def forward(cfg, w, tokens):
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    positions = list(range(T))
    x = w["embed"].to(F64)[torch.tensor(tokens)]
    S = cfg.get("streams")
    streams = [x.clone() for _ in range(S)] if S else [x]
    v_first = None
    per_layer = []
    for i, spec in enumerate(cfg["layers"]):
        pre = f"l{i}."
        assert spec["type"] == "attention"
        subs = [1] + ([2] if spec.get("mlp") else [])
        for q in subs:
            u = hyper_in(streams, w[f"{pre}hc{q}.in"]) if S else streams[0]
            hin = layer_norm(u, w[f"{pre}norm{q}"], eps)
            if q == 1:
                y, v_own = attention_mixer(hin, w, pre + "mix.", spec["mixer"], eps, positions, v_first)
                if spec["mixer"].get("v_mix") and v_first is None:
                    v_first = v_own
            elif spec["mlp"]["kind"] == "dense":
                y = dense_ff(hin, w, pre + "mlp.")
            else:
                y = moe_ff(hin, w, pre + "mlp.", spec["mlp"])
            if S:
                streams = hyper_out(streams, y, w[f"{pre}hc{q}.mix"], w[f"{pre}hc{q}.out"])
            else:
                streams = [streams[0] + y]
        per_layer.append(sum(streams))
    x = layer_norm(sum(streams), w["final.norm"], eps)
    return x @ w["head"].to(F64).T, torch.stack(per_layer)


def random_weights(cfg, seed=0):
    """Random bfloat16 tensors with the checkpoint's names and shapes. Nothing is left at a value
    that would hide a mechanism: stream mixes are far from the identity, biases and corrections
    are of the size of what they are added to, norm weights differ from 1."""
    g = torch.Generator().manual_seed(seed)
    d, V, S = cfg["width"], cfg["vocab"], cfg.get("streams")
    w = {}

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16)

    def lin(o, i):
        return rnd(o, i, std=1.0 / math.sqrt(i))

    w["embed"] = rnd(V, d)
    w["final.norm"] = rnd(d, std=0.2, mean=1.0)
    w["head"] = lin(V, d)
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for q in (1, 2) if spec.get("mlp") else (1,):
            w[f"{p}norm{q}"] = rnd(d, std=0.2, mean=1.0)
            if S:
                w[f"{p}hc{q}.in"] = rnd(S, std=0.5, mean=0.6)
                w[f"{p}hc{q}.out"] = rnd(S, std=0.5, mean=0.7)
                w[f"{p}hc{q}.mix"] = (torch.eye(S) * 0.8 + torch.randn(S, S, generator=g) * 0.3).to(torch.bfloat16)
        w[p + "mix.q"], w[p + "mix.q.b"] = lin(H * dim, d), rnd(H * dim, std=0.5)
        w[p + "mix.k"], w[p + "mix.k.b"] = lin(G * dim, d), rnd(G * dim, std=0.5)
        w[p + "mix.v"], w[p + "mix.v.b"] = lin(G * vdim, d), rnd(G * vdim, std=0.5)
        w[p + "mix.vmix"] = torch.tensor(0.2 + 0.6 * torch.rand((), generator=g).item()).to(torch.bfloat16)
        w[p + "mix.g"] = lin(H * vdim, d)
        w[p + "mix.o"] = lin(d, H * vdim)
        f = spec.get("mlp")
        if not f:
            continue
        if f["kind"] == "dense":
            w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = lin(f["ff"], d), lin(f["ff"], d), lin(d, f["ff"])
        else:
            r, ff = f["router"], f["expert"]["ff"]
            n = r["experts"] + r.get("identity", 0)
            w[p + "mlp.router"] = rnd(n, d, std=2.0 / math.sqrt(d))
            w[p + "mlp.correction"] = rnd(n, std=0.3)
            for e in range(r["experts"]):
                w[f"{p}mlp.e{e}.gate"], w[f"{p}mlp.e{e}.up"] = lin(ff, d), lin(ff, d)
                w[f"{p}mlp.e{e}.down"] = lin(d, ff)
    return w
