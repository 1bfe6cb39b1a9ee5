"""A plain, slow float64 implementation of the Mekusun design, one function per mechanism,
written from the design's equations. It shares no code with llmd_amd: the tests compare the
framework (CPU reference ops and HIP kernels, through the engine) against it.

Weights are a dict name -> tensor, named as in a checkpoint ('l<i>.mix.q', 'l<i>.mlp.e3.up', ...).
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_centered(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def gelu_erf(z):
    return 0.5 * z * (1 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def rotate(v, pos, dims, base):
    """v [T, ..., n]: rotate-half pairs (i, i + dims/2) over the first ``dims`` entries."""
    half = dims // 2
    f = torch.tensor(base, dtype=F64) ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    a = pos.to(F64)[:, None] * f[None]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    c, s = a.cos().view(shape), a.sin().view(shape)
    u, w = v[..., :half], v[..., half:dims]
    return torch.cat([u * c - w * s, w * c + u * s, v[..., dims:]], -1)


def attention_core(q, k, v, scale):
    """q [T, H, D], k [T, H, D], v [T, H, Dv], causal, ordinary softmax."""
    T = q.shape[0]
    s = torch.einsum("thd,shd->hts", q, k) * scale
    s = s.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), float("-inf"))
    return torch.einsum("hts,shd->thd", torch.softmax(s, -1), v)


def latent_attention(W, p, m, h, eps):
    T = h.shape[0]
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ W[p + "q"].T).view(T, H, dn + dr)
    kv = h @ W[p + "dkv"].T
    c = rms(kv[:, :R], eps) * W[p + "dkv.norm"]
    k_rot = rotate(kv[:, R:], pos, m["rot"]["dims"], m["rot"]["base"])
    q_rot = rotate(q[..., dn:], pos, m["rot"]["dims"], m["rot"]["base"])
    k = torch.cat([(c @ W[p + "uk"].T).view(T, H, dn), k_rot[:, None].expand(T, H, dr)], -1)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    o = attention_core(torch.cat([q[..., :dn], q_rot], -1), k, v, m["scale"])
    return o.reshape(T, H * dv) @ W[p + "o"].T


def mamba1(W, p, m, h):
    T = h.shape[0]
    C, N, R, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
    xz = h @ W[p + "in"].T
    x, z = xz[:, :C], xz[:, C:]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x])
    conv = W[p + "conv.b"].expand(T, C).clone()
    for j in range(taps):
        conv = conv + padded[j:j + T] * W[p + "conv"][:, j]
    x = silu(conv)
    proj = x @ W[p + "x"].T
    dt = softplus(proj[:, :R] @ W[p + "dt"].T + W[p + "dt.b"])
    B, Cm = proj[:, R:R + N], proj[:, R + N:R + 2 * N]
    A = -torch.exp(W[p + "A_log"])
    S = torch.zeros(C, N, dtype=F64)
    y = []
    for t in range(T):
        S = torch.exp(dt[t, :, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y.append(S @ Cm[t] + W[p + "D"] * x[t])
    return (torch.stack(y) * silu(z)) @ W[p + "o"].T


def general_delta(W, p, m, h, eps):
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    r, k, v = ((h @ W[p + n].T).view(T, H, d) for n in "rkv")
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"]))
    w = w.view(T, H, d)
    a = torch.sigmoid(h @ W[p + "a"].T + W[p + "a.b"]).view(T, H, d)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, d, d, dtype=F64)
    outs = []
    for t in range(T):
        old = S
        S = (w[t][:, :, None] * old - (a[t] * u[t])[:, :, None] * torch.einsum("hi,hij->hj", u[t], old)[:, None, :]
             + k[t][:, :, None] * v[t][:, None, :])
        outs.append(torch.einsum("hij,hi->hj", S, r[t]))
    o = rms(torch.stack(outs), eps).reshape(T, H * d)
    return (o * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def xielu(z, pq):
    sp, sq = softplus(pq[0]), softplus(pq[1])
    return torch.where(z > 0, sp * z * z + z / 2, (0.5 + sq) * (torch.exp(z) - 1 - z) + z / 2)


def dense_ff(W, p, h):
    return xielu(h @ W[p + "up"].T, W[p + "act"]) @ W[p + "down"].T


def moe_ff(W, p, m, h):
    k = m["router"]["top"]
    z = h @ W[p + "router"].T + W[p + "router.b"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = sorted(range(z.shape[1]), key=lambda e: (-float(z[t, e]), e))[:k]
        wts = torch.softmax(z[t, chosen], -1)
        for wt, e in zip(wts, chosen):
            out[t] += wt * (gelu_erf(h[t] @ W[f"{p}e{e}.up"].T) @ W[f"{p}e{e}.down"].T)
    return out


def forward(cfg, W, tokens, streams=None):
    """Logits [T, vocab] of one sequence; ``streams`` (a list) receives the stream after every layer."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    X = [x]
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = norm_centered(x, W[pre + "norm1"], eps)
        if L["type"] == "latent_attention":
            y = latent_attention(W, pre + "mix.", L["mixer"], h, eps)
        elif L["type"] == "mamba1":
            y = mamba1(W, pre + "mix.", L["mixer"], h)
        else:
            y = general_delta(W, pre + "mix.", L["mixer"], h, eps)
        x = x + norm_centered(y, W[pre + "norm1b"], eps) * W[pre + "ls1"]
        if L.get("mlp"):
            h = norm_centered(x, W[pre + "norm2"], eps)
            y = dense_ff(W, pre + "mlp.", h) if L["mlp"]["kind"] == "dense" else moe_ff(W, pre + "mlp.", L["mlp"], h)
            x = x + norm_centered(y, W[pre + "norm2b"], eps) * W[pre + "ls2"]
        X.append(x)
        x = sum(W[pre + "dwa"][j] * X[j] for j in range(i + 2))
        if streams is not None:
            streams.append(x)
    z = norm_centered(x, W["final.norm"], eps) @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


def random_weights(cfg, seed, decay_rank=8):
    """Random bfloat16 weights with every tensor a checkpoint of ``cfg`` has."""
    g = torch.Generator().manual_seed(seed)
    d, V = cfg["width"], cfg["vocab"]
    W = {}

    def lin(name, out, inp, gain=1.0):
        W[name] = torch.randn(out, inp, generator=g) * (gain / math.sqrt(inp))

    def vec(name, n, std=0.1, mean=0.0):
        W[name] = torch.randn(n, generator=g) * std + mean

    W["embed"] = torch.randn(V, d, generator=g) * 0.5
    lin("head", V, d)
    vec("final.norm", d)
    for i, L in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", L["mixer"]
        for n in ("norm1", "norm1b"):
            vec(pre + n, d)
        vec(pre + "ls1", d, 0.1, 0.8)
        W[pre + "dwa"] = torch.softmax(torch.randn(i + 2, generator=g), 0) + 0.1 * torch.randn(i + 2, generator=g)
        p = pre + "mix."
        if L["type"] == "latent_attention":
            H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            lin(p + "q", H * (dn + dr), d, 2.0)
            lin(p + "dkv", R + dr, d, 2.0)
            vec(p + "dkv.norm", R, 0.1, 1.0)
            lin(p + "uk", H * dn, R, 2.0)
            lin(p + "uv", H * dv, R)
            lin(p + "o", d, H * dv)
        elif L["type"] == "mamba1":
            C, N, R, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
            lin(p + "in", 2 * C, d)
            W[p + "conv"] = torch.randn(C, taps, generator=g) * 0.5
            vec(p + "conv.b", C)
            lin(p + "x", R + 2 * N, C)
            lin(p + "dt", C, R)
            vec(p + "dt.b", C, 0.5, -1.0)
            W[p + "A_log"] = torch.log(torch.rand(C, N, generator=g) * 4 + 0.2)
            vec(p + "D", C, 0.3, 1.0)
            lin(p + "o", d, C)
        else:
            HD = m["heads"] * m["dim"]
            for n in "rkvga":
                lin(p + n, HD, d)
            vec(p + "a.b", HD, 0.3)
            lin(p + "w1", decay_rank, d)
            lin(p + "w2", HD, decay_rank)
            vec(p + "w0", HD, 0.5)
            vec(p + "norm", HD, 0.1, 1.0)
            lin(p + "o", d, HD)
        f = L.get("mlp")
        if f:
            for n in ("norm2", "norm2b"):
                vec(pre + n, d)
            vec(pre + "ls2", d, 0.1, 0.8)
            p = pre + "mlp."
            if f["kind"] == "dense":
                lin(p + "up", f["ff"], d)
                lin(p + "down", d, f["ff"])
                vec(p + "act", 2, 0.5)
            else:
                E = f["router"]["experts"]
                lin(p + "router", E, d, 3.0)
                vec(p + "router.b", E, 0.3)
                for e in range(E):
                    lin(f"{p}e{e}.up", f["expert"]["ff"], d)
                    lin(f"{p}e{e}.down", d, f["expert"]["ff"])
    return {k: v.to(torch.bfloat16) for k, v in W.items()}
