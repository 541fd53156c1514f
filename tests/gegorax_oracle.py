"""Plain, slow oracle for the Gegorax design (one function per mechanism).

Written from the design's equations in double precision, one token at a time
where the design is recurrent; shares no code with ``dnet_amd``. ``cfg`` is
the checkpoint's config.json as a dict, ``sd`` maps checkpoint tensor names to
tensors.

A layer: u = rms(x) g;  x <- x + mixer(u) + ff(u);  then the per-layer token
input x <- x + rms(P (gelu(G x) * e_tok)) s, with e_tok the layer's slice of a
second embedding row of the token.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(x.clamp(max=30.0))))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


# ---------- attention with a window and pooled blocks ----------

def rotate(x, pos, rot):
    """x [T, heads, d]; interleaved pairs (2i, 2i+1) of the first rot.dims
    channels turn by pos * base^(-2i/dims)."""
    if not rot:
        return x
    n, base = int(rot["dims"]), float(rot["base"])
    out = x.clone()
    for i in range(n // 2):
        a = pos.to(F64) * base ** (-2.0 * i / n)
        c, s = torch.cos(a).view(-1, 1), torch.sin(a).view(-1, 1)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def visible(i, size, pool):
    """(token positions, pooled block ids) that query position i sees."""
    if not size:
        return list(range(i + 1)), []
    toks = [j for j in range(i + 1) if i - j < size]
    blocks = []
    if pool:
        b = 0
        while b * pool + pool - 1 <= i - size:
            blocks.append(b)
            b += 1
    return toks, blocks


def window_pool_attention(q, k, v, scale, size, pool):
    """q [T, H, d], k [T, G, d], v [T, G, dv] (k as cached: normalized and
    rotated). Tokens inside the window and the means of whole blocks before
    it share one softmax."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for i in range(T):
        toks, blocks = visible(i, size, pool)
        for h in range(H):
            g = h // (H // G)
            ks = [k[j, g] for j in toks] + \
                 [k[b * pool:(b + 1) * pool, g].mean(0) for b in blocks]
            vs = [v[j, g] for j in toks] + \
                 [v[b * pool:(b + 1) * pool, g].mean(0) for b in blocks]
            K, V = torch.stack(ks), torch.stack(vs)
            p = torch.softmax((K @ q[i, h]) * scale, dim=0)
            out[i, h] = p @ V
    return out


def attention(u, w, m, eps, pre):
    T = u.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (u @ w[pre + "q"].T).view(T, H, d)
    k = (u @ w[pre + "k"].T).view(T, G, d)
    v = (u @ w[pre + "v"].T).view(T, G, dv)
    q = rms(q, eps) * w[pre + "q.norm"]
    k = rms(k, eps) * w[pre + "k.norm"]
    pos = torch.arange(T)
    q, k = rotate(q, pos, m.get("rot")), rotate(k, pos, m.get("rot"))
    mask = m.get("mask") or {}
    o = window_pool_attention(q, k, v, float(m["scale"]),
                              int(mask.get("size") or 0),
                              int(mask.get("pool") or 0))
    return o.reshape(T, H * dv) @ w[pre + "o"].T


# ---------- selective state space (scalar decay per head) ----------

def causal_conv(x, cw, cb):
    """x [T, C]; cw [C, taps], last column = current token; zeros before 0."""
    T, C = x.shape
    taps = cw.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x])
    out = cb.expand(T, C).clone()
    for j in range(taps):
        out = out + xp[j:j + T] * cw[:, j]
    return out


def ssd(u, w, m, eps, pre):
    T = u.shape[0]
    Hh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = Hh * P
    zz = u @ w[pre + "in"].T
    z, xbc, dt = zz[:, :inner], zz[:, inner:2 * inner + 2 * G * N], \
        zz[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[pre + "conv"], w[pre + "conv.b"]))
    x = xbc[:, :inner].view(T, Hh, P)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[pre + "dt_bias"])
    y = torch.zeros(T, Hh, P, dtype=F64)
    for h in range(Hh):
        g = h // (Hh // G)
        S = torch.zeros(N, P, dtype=F64)
        decay = torch.exp(w[pre + "A_log"][h])
        for t in range(T):
            S = torch.exp(-decay * dt[t, h]) * S + \
                dt[t, h] * torch.outer(Bm[t, g], x[t, h])
            y[t, h] = S.T @ Cm[t, g] + w[pre + "D"][h] * x[t, h]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * w[pre + "norm"]
    return y @ w[pre + "o"].T


def parallel_mixer(u, w, m, eps):
    a = attention(u, w, m["left"], eps, "mix.left.")
    b = ssd(u, w, m["right"], eps, "mix.right.")
    return 0.5 * (rms(a, eps) * w["mix.left.out"]
                  + rms(b, eps) * w["mix.right.out"])


# ---------- generalized delta rule ----------

def general_delta(u, w, m, eps):
    T = u.shape[0]
    H, d = m["heads"], m["dim"]
    r = (u @ w["mix.r"].T).view(T, H, d)
    k = (u @ w["mix.k"].T).view(T, H, d)
    v = (u @ w["mix.v"].T).view(T, H, d)
    dec = torch.exp(-math.exp(-0.5) * sigmoid(
        torch.tanh(u @ w["mix.w1"].T) @ w["mix.w2"].T + w["mix.w0"])
    ).view(T, H, d)
    a = sigmoid(u @ w["mix.a"].T + w["mix.a.b"]).view(T, H, d)
    o = torch.zeros(T, H, d, dtype=F64)
    for h in range(H):
        S = torch.zeros(d, d, dtype=F64)
        for t in range(T):
            kk = k[t, h]
            un = kk / torch.sqrt((kk * kk).sum() + 1e-6)
            S = dec[t, h].view(d, 1) * S \
                - torch.outer(a[t, h] * un, un @ S) + torch.outer(kk, v[t, h])
            o[t, h] = S.T @ r[t, h]
    o = rms(o, eps).reshape(T, H * d) * w["mix.norm"]
    o = o * sigmoid(u @ w["mix.g"].T)
    return o @ w["mix.o"].T


# ---------- feed-forwards ----------

def dense_ff(u, w):
    return torch.relu(u @ w["mlp.up"].T) ** 2 @ w["mlp.down"].T


def clamped_glu_expert(u, w, pre, limit):
    g = (u @ w[pre + "gate"].T).clamp(max=limit)
    up = (u @ w[pre + "up"].T).clamp(min=-limit, max=limit)
    return (g * sigmoid(1.702 * g) * (up + 1.0)) @ w[pre + "down"].T


def route(u, w, top):
    z = u @ w["mlp.router"].T + w["mlp.router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    return torch.softmax(val, dim=-1), idx


def moe_ff(u, w, ff):
    T = u.shape[0]
    top = ff["router"]["top"]
    wt, idx = route(u, w, top)
    out = torch.zeros(T, w["mlp.e0.down"].shape[0], dtype=F64)
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            out[t] += wt[t, j] * clamped_glu_expert(
                u[t:t + 1], w, f"mlp.e{e}.", float(ff["expert"]["limit"]))[0]
    if ff.get("shared"):
        out = out + clamped_glu_expert(u, w, "mlp.shared.",
                                       float(ff["shared"]["limit"]))
    return out


def token_side(x, tokens, li, w, side_embed, dim, eps):
    e = side_embed[tokens][:, li * dim:(li + 1) * dim]
    g = gelu_tanh(x @ w["side.gate"].T) * e
    y = g @ w["side.proj"].T
    return x + rms(y, eps) * w["side.norm"]


# ---------- the model ----------

def layer_weights(sd, i):
    p = f"l{i}."
    return {k[len(p):]: v.to(F64) for k, v in sd.items() if k.startswith(p)}


def forward(tokens, cfg, sd, residuals=None):
    """Logits [T, vocab] (float64) of one sequence; ``residuals`` (a list)
    receives the residual stream after every layer."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = float(cfg["norm"]["eps"])
    x = sd["embed"].to(F64)[tokens]
    side = cfg.get("token_side")
    for i, spec in enumerate(cfg["layers"]):
        w = layer_weights(sd, i)
        u = rms(x, eps) * w["norm1"]
        if spec["type"] == "parallel":
            mix = parallel_mixer(u, w, spec["mixer"], eps)
        elif spec["type"] == "general_delta":
            mix = general_delta(u, w, spec["mixer"], eps)
        else:
            raise ValueError(spec["type"])
        ff = spec.get("mlp")
        if ff is None:
            x = x + mix
        elif ff["kind"] == "dense":
            x = x + (mix + dense_ff(u, w))
        else:
            x = x + (mix + moe_ff(u, w, ff))
        if side:
            x = token_side(x, tokens, i, w, sd["side.embed"].to(F64),
                           int(side["dim"]), eps)
        if residuals is not None:
            residuals.append(x.clone())
    return (rms(x, eps) * sd["final.norm"].to(F64)) @ sd["head"].to(F64).T
