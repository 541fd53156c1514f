"""Plain, slow oracle for the Posudra design (one function per mechanism).

Written directly from the design's equations in double precision; shares no
code with ``dnet_amd``. Layers are dicts of torch tensors keyed by the
checkpoint's tensor names without the ``l<i>.`` prefix.

Notation: x residual stream [T, W]; a layer computes
    u = rms(x) * g                      (one norm feeds both branches)
    x <- x + s1 * attn(u) + s2 * ff(u)  (s1, s2 element-wise layer scales)
"""
from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def softplus(t: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(t))


def xielu(z: torch.Tensor, p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    """z>0: softplus(p) z^2 + z/2 ; z<=0: (1/2+softplus(q)) (e^z - 1 - z) + z/2."""
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (torch.exp(z.clamp(max=0.0)) - 1.0 - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def feed_forward(u, w):
    z = u @ w["mlp.up"].T
    a = xielu(z, w["mlp.act"][0], w["mlp.act"][1])
    return a @ w["mlp.down"].T


def attention_scores(q, k, head, mx, w):
    """Pre-softmax logits [T, T] of one query head (q [T,d], k [T,d]),
    causal entries only meaningful."""
    T = q.shape[0]
    s = (q @ k.T) * mx["scale"] * w["mix.temp"][head]
    cap = mx.get("softcap")
    if cap:
        s = cap * torch.tanh(s / cap)
    i = torch.arange(T, dtype=s.dtype).view(T, 1)
    j = torch.arange(T, dtype=s.dtype).view(1, T)
    dist = (i - j).clamp(min=0.0)
    return s - w["mix.r1"][head] * torch.log1p(w["mix.r2"][head] * dist)


def sink_softmax(s, sink):
    """Row softmax over causal entries of s [T,T] whose denominator also
    holds exp(sink) (a slot with no key and no value)."""
    T = s.shape[0]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    s = s.masked_fill(~mask, -math.inf)
    m = torch.maximum(s.max(dim=-1, keepdim=True).values, sink)
    e = torch.exp(s - m)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - m))


def attention(u, w, mx, eps):
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    T = u.shape[0]
    q = rms(u @ w["mix.q"].T, eps) * w["mix.q.norm"]      # norm over all heads at once
    k = rms(u @ w["mix.k"].T, eps) * w["mix.k.norm"]
    v = u @ w["mix.v"].T
    q = q.view(T, H, d)
    k = k.view(T, G, d)
    v = v.view(T, G, dv)
    outs = []
    for h in range(H):
        g = h // (H // G)
        s = attention_scores(q[:, h], k[:, g], h, mx, w)
        p = sink_softmax(s, w["mix.sink"][h])
        outs.append(p @ v[:, g])
    return torch.cat(outs, dim=-1) @ w["mix.o"].T


def layer(x, w, spec, eps):
    u = rms(x, eps) * w["norm1"]
    y = w["ls1"] * attention(u, w, spec["mixer"], eps)
    if spec.get("mlp") is not None:
        y = y + w["ls2"] * feed_forward(u, w)
    return x + y


def forward(tokens, cfg, sd, dtype=torch.float64, return_layers=False):
    """Logits [T, V] for one sequence; sd maps checkpoint names to tensors."""
    sd = {n: t.to(dtype) for n, t in sd.items()}
    eps = cfg["norm"]["eps"]
    x = sd["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    trail = []
    for i, spec in enumerate(cfg["layers"]):
        assert spec["type"] == "attention"
        pre = f"l{i}."
        w = {n[len(pre):]: t for n, t in sd.items() if n.startswith(pre)}
        x = layer(x, w, spec, eps)
        trail.append(x)
    y = rms(x, eps) * sd["final.norm"]
    logits = y @ sd["head"].T
    return (logits, torch.stack(trail)) if return_layers else logits
