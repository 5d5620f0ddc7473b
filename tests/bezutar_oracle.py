"""Plain, slow, per-sequence implementation of the Bezutar design (test oracle).

One function per mechanism, written directly from the design's equations; it
shares no code with the framework's product path (no ragged batches, no pages,
no state slots, no fused projections, no absorbed attention): whole sequences,
token by token, every key and value recomputed from the start.  Weights are
addressed by their checkpoint names.
"""
import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def softplus(x):
    return math.log1p(math.exp(-abs(x))) + max(x, 0.0)


def xielu(z, p, q):
    ap = softplus(float(p))
    aq = 0.5 + softplus(float(q))
    pos = ap * z * z + z / 2
    neg = aq * (torch.exp(torch.clamp(z, max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def embed_tokens(W, cfg, tokens, dt):
    T = len(tokens)
    x = W["embed"].to(dt)[torch.tensor(tokens)]
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        rows = []
        for t in range(T):
            if t == 0:
                rows.append(bg["buckets"])
            else:
                rows.append((tokens[t - 1] * bg["mul_prev"] + tokens[t] * bg["mul_cur"]) % bg["buckets"])
        x = x + W["bigram"].to(dt)[torch.tensor(rows)]
    if "pos" in W:
        x = x + W["pos"].to(dt)[:T]
    return x


def canon_conv(h, w):
    """h [T, C], w [C, taps]: out_t = sum_j w[:, j] h_{t-taps+1+j}."""
    T, C = h.shape
    taps = w.shape[1]
    out = torch.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def yarn_tables(rot, T, dt):
    dims = rot["dims"]
    base = rot["base"]
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    mscale = 1.0
    sc = rot.get("scaling")
    if sc:
        def dim_of(t):
            return dims * math.log(sc["original"] / (2 * math.pi * t)) / (2 * math.log(base))
        lo = max(math.floor(dim_of(sc["fast"])), 0)
        hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
        ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=torch.float64)
        f = f / sc["factor"] * ramp + f * (1 - ramp)
        mscale = 0.1 * math.log(sc["factor"]) + 1.0
    f = f.to(torch.float32)
    ang = torch.arange(T, dtype=torch.float32)[:, None] * f[None, :]
    return (torch.cos(ang) * mscale).to(dt), (torch.sin(ang) * mscale).to(dt)


def rotate(x, cos, sin, dims):
    """x [T, ..., D]; rotate first dims, pair i with i + dims/2."""
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = cos.view(shape), sin.view(shape)
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def latent_kv(W, pre, m, h, eps, dt):
    """The cached part: normed latent c [T, r] and rotated shared key part [T, rot_dim]."""
    T = h.shape[0]
    r, rd = m["kv_rank"], m["rot_dim"]
    d = h @ W[pre + "dkv"].to(dt).T
    c = rms(d[:, :r], eps) * W[pre + "dkv.norm"].to(dt)
    kr = d[:, r:]
    cos, sin = yarn_tables(m["rot"], T, dt)
    kr = rotate(kr, cos, sin, m["rot"]["dims"])
    return c, kr


def latent_attention(W, pre, m, h, eps, dt, shared):
    T = h.shape[0]
    H, D, rd, vd = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = rms(h @ W[pre + "dq"].to(dt).T, eps) * W[pre + "dq.norm"].to(dt)
    q = (cq @ W[pre + "uq"].to(dt).T).view(T, H, D + rd)
    qn, qr = q[..., :D], q[..., D:]
    cos, sin = yarn_tables(m["rot"], T, dt)
    qr = rotate(qr, cos, sin, m["rot"]["dims"])
    c, kr = shared
    kn = (c @ W[pre + "uk"].to(dt).T).view(T, H, D)
    v = (c @ W[pre + "uv"].to(dt).T).view(T, H, vd)
    sink = W[pre + "sink"].to(dt)
    gate = torch.sigmoid(h @ W[pre + "g"].to(dt).T)  # [T, H]
    out = torch.zeros(T, H, vd, dtype=dt)
    for t in range(T):
        for hh in range(H):
            s = (kn[: t + 1, hh] @ qn[t, hh] + kr[: t + 1] @ qr[t, hh]) * m["scale"]
            mx = torch.maximum(s.max(), sink[hh])
            e = torch.exp(s - mx)
            den = e.sum() + torch.exp(sink[hh] - mx)
            out[t, hh] = (e[:, None] * v[: t + 1, hh]).sum(0) / den * gate[t, hh]
    return out.reshape(T, H * vd) @ W[pre + "o"].to(dt).T


def mlstm(W, pre, m, h, eps, dt):
    T = h.shape[0]
    H, D, vd, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ W[pre + "q"].to(dt).T).view(T, H, D) * D ** -0.5
    k = (h @ W[pre + "k"].to(dt).T).view(T, H, D)
    v = (h @ W[pre + "v"].to(dt).T).view(T, H, vd)
    ig = cap * torch.tanh((h @ W[pre + "i"].to(dt).T + W[pre + "i.b"].to(dt)) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W[pre + "f"].to(dt).T + W[pre + "f.b"].to(dt)) / cap))
    S = torch.zeros(H, D, vd, dtype=dt)
    n = torch.zeros(H, D, dtype=dt)
    mm = torch.zeros(H, dtype=dt)
    o = torch.zeros(T, H, vd, dtype=dt)
    for t in range(T):
        m_new = torch.maximum(fg[t] + mm, ig[t])
        a = torch.exp(fg[t] + mm - m_new)
        b = torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mm = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mm)) + 1e-6
        o[t] = num / den[:, None]
    o = rms(o, eps).reshape(T, H * vd) * W[pre + "norm"].to(dt)
    o = o * torch.sigmoid(h @ W[pre + "g"].to(dt).T)
    return o @ W[pre + "o"].to(dt).T


def mingru(W, pre, m, h, dt):
    T = h.shape[0]
    z = torch.sigmoid(h @ W[pre + "z"].to(dt).T + W[pre + "z.b"].to(dt))
    u = h @ W[pre + "x"].to(dt).T + W[pre + "x.b"].to(dt)
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(m["width"], dtype=dt)
    out = torch.zeros(T, m["width"], dtype=dt)
    for t in range(T):
        S = (1 - z[t]) * S + z[t] * cand[t]
        out[t] = S
    out = out * torch.nn.functional.silu(h @ W[pre + "g"].to(dt).T)
    return out @ W[pre + "o"].to(dt).T


def dense_ff(W, pre, h, dt):
    a = W[pre + "act"].to(torch.float32)
    return xielu(h @ W[pre + "up"].to(dt).T, a[0], a[1]) @ W[pre + "down"].to(dt).T


def norm_w(x, w, eps):
    return rms(x, eps) * (1 + w)


def forward(W, cfg, tokens, dt=torch.float32, layers_out=None):
    eps = cfg["norm"]["eps"]
    x0 = embed_tokens(W, cfg, tokens, dt)
    ns = cfg.get("streams")
    xs = [x0.clone() for _ in range(ns)] if ns else [x0]
    caches = {}
    for li, L in enumerate(cfg["layers"]):
        p = "l%d." % li
        for q in (1, 2):
            if q == 2 and not L.get("mlp"):
                continue
            if ns:
                hin = W[p + "hc%d.in" % q].to(dt)
                u = sum(hin[s] * xs[s] for s in range(ns))
            else:
                u = xs[0]
            h = norm_w(u, W[p + "norm%d" % q].to(dt), eps)
            if q == 1:
                if cfg.get("canon"):
                    h = h + canon_conv(h, W[p + "canon1"].to(dt))
                m = L["mixer"]
                if L["type"] == "latent_attention":
                    if "kv_from" in m and m["kv_from"] is not None:
                        shared = caches[m["kv_from"]]
                    else:
                        shared = caches[li] = latent_kv(W, p + "mix.", m, h, eps, dt)
                    y = latent_attention(W, p + "mix.", m, h, eps, dt, shared)
                elif L["type"] == "mlstm":
                    y = mlstm(W, p + "mix.", m, h, eps, dt)
                elif L["type"] == "mingru":
                    y = mingru(W, p + "mix.", m, h, dt)
                else:
                    raise ValueError(L["type"])
            else:
                y = dense_ff(W, p + "mlp.", h, dt)
            if ns:
                mix = W[p + "hc%d.mix" % q].to(dt)
                hout = W[p + "hc%d.out" % q].to(dt)
                xs = [sum(mix[s, t] * xs[s] for s in range(ns)) + hout[t] * y for t in range(ns)]
            else:
                xs = [xs[0] + y]
        if layers_out is not None:
            layers_out.append(sum(xs))
    x = sum(xs)
    x = norm_w(x, W["final.norm"].to(dt), eps)
    return x @ W["head"].to(dt).T
