"""Plain, slow, per-sequence implementation of the Bezurax design in fp32
(fp64 on request), one function per mechanism, written from the design's
equations.  It shares no code with megatron_amd: the tests compare the
framework against it.

Weights are a dict name -> tensor with the checkpoint's names; the config is
the config.json dict.
"""

from __future__ import annotations

import math

import torch


def group_rms_norm(x, w, groups, eps):
    """x [n, W]: each of ``groups`` consecutive parts is divided by its own
    root mean square; the whole is multiplied by w."""
    n, W = x.shape
    p = x.view(n, groups, W // groups)
    p = p / torch.sqrt((p * p).mean(-1, keepdim=True) + eps)
    return p.reshape(n, W) * w


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def pooled_window_attention(h, W, pre, m, eps):
    """Left mixer: grouped-query attention, values = raw keys, whole-projection
    q/k norm, no rotation, sliding window plus mean-pooled blocks before it."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size, P = m["mask"]["size"], m["mask"]["pool"]
    q = h @ W[pre + "q"].T
    k = h @ W[pre + "k"].T
    v = k.clone().view(n, G, V)
    q = (rms(q, eps) * W[pre + "q.norm"]).view(n, H, D)
    k = (rms(k, eps) * W[pre + "k.norm"]).view(n, G, D)
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for i in range(n):
        lo = max(0, i - size + 1)
        keys = [k[j] for j in range(lo, i + 1)]
        vals = [v[j] for j in range(lo, i + 1)]
        b = 0
        while b * P + P - 1 <= i - size:
            keys.append(k[b * P:b * P + P].mean(0))
            vals.append(v[b * P:b * P + P].mean(0))
            b += 1
        K = torch.stack(keys)            # [L, G, D]
        Vv = torch.stack(vals)           # [L, G, V]
        for hd in range(H):
            g = hd // (H // G)
            s = (K[:, g] @ q[i, hd]) * m["scale"]
            p = torch.softmax(s, dim=0)
            out[i, hd] = p @ Vv[:, g]
    return out.reshape(n, H * V) @ W[pre + "o"].T


def delta_rule(h, W, pre, m, eps):
    """Right mixer: generalized delta rule with per-channel decay and removal."""
    n = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (h @ W[pre + "r"].T).view(n, H, D)
    k = (h @ W[pre + "k"].T).view(n, H, D)
    v = (h @ W[pre + "v"].T).view(n, H, D)
    z = torch.tanh(h @ W[pre + "w1"].T) @ W[pre + "w2"].T + W[pre + "w0"]
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(z)).view(n, H, D)
    a = torch.sigmoid(h @ W[pre + "a"].T + W[pre + "a.b"]).view(n, H, D)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, D, D, dtype=h.dtype)
    o = torch.zeros(n, H, D, dtype=h.dtype)
    for t in range(n):
        uS = torch.einsum("hd,hde->he", u[t], S)
        S = w[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hde,hd->he", S, r[t])
    o = rms(o, eps).reshape(n, H * D) * W[pre + "norm"] * torch.sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def expert(h, W, pre, limit):
    g = torch.clamp(h @ W[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ W[pre + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ W[pre + "down"].T


def route(h, W, pre, rt):
    """-> (chosen experts [n, top], weights [n, top])"""
    s = torch.sigmoid(h @ W[pre + "router"].T)
    n, E = s.shape
    top = rt["top"]
    gr = rt.get("groups")
    allowed = torch.ones(n, E, dtype=torch.bool)
    if gr and gr["count"] > 1:
        cnt, keep = gr["count"], gr["keep"]
        per = E // cnt
        gs = s.view(n, cnt, per).topk(min(2, per), dim=-1).values.sum(-1)
        best = gs.topk(keep, dim=-1).indices
        allowed = torch.zeros(n, cnt, dtype=torch.bool)
        allowed.scatter_(1, best, True)
        allowed = allowed[:, :, None].expand(n, cnt, per).reshape(n, E)
    idx = s.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
    sc = s.gather(1, idx)
    wt = sc / (sc.sum(-1, keepdim=True) + 1e-20) * rt["scale"]
    return idx, wt


def moe(h, W, pre, mlp):
    n = h.shape[0]
    idx, wt = route(h, W, pre, mlp["router"])
    out = torch.zeros(n, W[pre + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(n):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            out[t] += wt[t, j] * expert(h[t:t + 1], W, f"{pre}e{e}.", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        sg = torch.sigmoid(h @ W[pre + "shared.sg"].T)           # [n, 1]
        out = out + sg * expert(h, W, pre + "shared.", mlp["shared"]["limit"])
    return out


def forward(cfg, W, tokens, trace=None, dtype=torch.float32):
    """tokens: list of ids of ONE sequence -> logits [n, vocab]."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, spec in enumerate(cfg["layers"]):
        p = "l%d." % spec.get("weights_of", i)
        assert spec["type"] == "parallel"
        m = spec["mixer"]
        h1 = group_rms_norm(x, W[p + "norm1"], groups, eps)
        y = (m["left_scale"] * pooled_window_attention(h1, W, p + "mix.left.", m["left"], eps)
             + m["right_scale"] * delta_rule(h1, W, p + "mix.right.", m["right"], eps))
        if spec.get("mlp"):
            h2 = group_rms_norm(x, W[p + "norm2"], groups, eps)
            y = y + moe(h2, W, p + "mlp.", spec["mlp"])
        x = x + y
        if trace is not None:
            trace.append(x.clone())
    x = group_rms_norm(x, W["final.norm"], groups, eps)
    return (x @ W["embed"].T) * cfg["logit_scale"]
