"""Posudra ring model: parallel-branch decoder with an fp32 residual stream.

Each layer normalizes the residual once and feeds both branches from it:

    u = rmsnorm(x) * g
    x <- x + s1 * attention(u) + s2 * feed_forward(u)       (x kept in fp32)

with element-wise layer scales s1, s2. The attention has no rotation; the
position enters the score only through a per-head logarithmic distance
penalty:

    s_ij = cap * tanh((q_i . k_j) * scale * temp_h / cap) - r1_h * ln(1 + r2_h (i - j))

q and k are RMS-normalized over the WHOLE projection (all heads at once,
plain weights) before they are split into heads, the key/value head sizes
may differ, and the softmax denominator carries one extra term exp(sink_h)
that has no key and no value. The feed-forward is up -> xIELU -> down.

Every size is per layer (``cfg.layer_specs``), so the KV cache is a list of
per-layer tensors. Checkpoint names: ``embed``, ``l<i>.norm1``,
``l<i>.mix.{q,k,v,o,q.norm,k.norm,temp,r1,r2,sink}``,
``l<i>.mlp.{up,down,act}``, ``l<i>.ls1``, ``l<i>.ls2``, ``final.norm``,
``head``.

Compute path (ops/__init__.py): one fused residual-update+norm kernel per
layer boundary, the fused projection [q;k;v], a fused q/k-norm + cache
append, the score-modified flash attention (decode and ragged prefill in
one entry point), the activation kernel, and the framework's GEMV/GEMM
linears. ``cfg.compute_dtype == "float32"`` runs weights, activations, the
cache and every product in true fp32.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from .. import ops
from .base import KVCache, LayerWeights, Linear, RingModel
from .config import ModelConfig


class PosudraRingModel(RingModel):
    model_type = "posudra"
    model_types = ["posudra"]
    act_dtype = torch.float32          # residual stream / ring hops
    ragged_prefill = True
    supports_float32 = True

    def __init__(self, cfg: ModelConfig, layer_ids: Sequence[int], device,
                 is_first: bool, is_last: bool, smax: int = 4096, **kw):
        if kw.get("tp_size", 1) > 1 or kw.get("cp_size", 1) > 1:
            # the whole-projection q/k norm needs every head's sum of
            # squares on one rank
            raise NotImplementedError(
                "posudra: tensor/context parallelism inside a stage is not "
                "implemented (pipeline stages are)")
        assert cfg.layer_specs is not None, "posudra needs per-layer specs"
        assert cfg.quant is None or cfg.quant.fmt != "mxfp4", \
            "posudra: grouped int8/int4 weights only"
        super().__init__(cfg, layer_ids, device, is_first, is_last,
                         smax=smax, **kw)
        self.wdtype = (torch.float32 if cfg.compute_dtype == "float32"
                       else torch.bfloat16)
        self.logits_dtype = self.wdtype

    def _init_positional(self):
        pass        # no rotation tables: distance enters inside the kernel

    # ---------- per-layer sizes ----------

    def _dims(self, lid: int):
        m = self.cfg.layer_specs[lid]["mixer"]
        return m["heads"], m["kv_heads"], m["dim"], m["vdim"]

    def _ff(self, lid: int) -> int:
        ff = self.cfg.layer_specs[lid].get("mlp")
        return 0 if ff is None else int(ff["ff"])

    def make_kv_cache(self, batch: int, smax: int) -> KVCache:
        dims = [self._dims(l)[1:] for l in self.layer_ids]
        return KVCache(self.cfg, self.layer_ids, batch, smax, self.device,
                       layer_dims=dims, dtype=self.wdtype)

    # ---------- weights ----------

    def _lin(self, w: torch.Tensor) -> Linear:
        q = self.cfg.quant
        if (q is not None and self.wdtype == torch.bfloat16
                and w.shape[1] % max(q.group, 128) == 0):
            # grouped int8/int4 weights through the framework's fused
            # dequant GEMMs (projections whose K does not fit stay bf16)
            return Linear.make(w.to(torch.bfloat16).to(self.device)
                               .contiguous(), None, q)
        return Linear(w.to(self.wdtype).to(self.device).contiguous())

    def _vec(self, t: torch.Tensor) -> torch.Tensor:
        # small per-channel / per-head parameters feed fp32 math directly
        return t.to(torch.float32).to(self.device).contiguous()

    def _build_layer(self, lid: int, get) -> LayerWeights:
        nq, nkv, d, dv = self._dims(lid)
        q, k, v = get("mix.q"), get("mix.k"), get("mix.v")
        assert q.shape[0] == nq * d and k.shape[0] == nkv * d \
            and v.shape[0] == nkv * dv, f"layer {lid}: projection shapes"
        lw = LayerWeights(
            attn_norm=self._vec(get("norm1")),
            qkv=self._lin(torch.cat([q, k, v])),
            o=self._lin(get("mix.o")),
            q_norm=self._vec(get("mix.q.norm")),
            k_norm=self._vec(get("mix.k.norm")),
            sinks=self._vec(get("mix.sink")),
        )
        lw.temp = self._vec(get("mix.temp"))
        lw.dist_r1 = self._vec(get("mix.r1"))
        lw.dist_r2 = self._vec(get("mix.r2"))
        lw.ls1 = self._vec(get("ls1"))
        lw.up = lw.act_pq = lw.ls2 = None
        if self._ff(lid):
            lw.up = self._lin(get("mlp.up"))
            lw.down = self._lin(get("mlp.down"))
            lw.act_pq = self._vec(get("mlp.act"))
            lw.ls2 = self._vec(get("ls2"))
        return lw

    def load_state_dict(self, sd: dict):
        for lid in self.layer_ids:
            self.layers[lid] = self._build_layer(
                lid, lambda n, p=f"l{lid}.": sd[p + n])
        if self.is_first:
            self.embed = sd["embed"].to(self.wdtype).to(self.device)
        if self.is_last:
            self.final_norm = self._vec(sd["final.norm"])
            self.lm_head = self._lin(sd["head"])

    def init_random(self, seed: int = 0):
        """Seeded per layer id (any sharding of one (model, seed) holds the
        same global weights). Scales are chosen so that every mechanism —
        sink, distance penalty, soft cap, both activation branches — moves
        the logits."""
        c = self.cfg
        W = c.hidden_size

        on_gpu = self.device.type == "cuda"
        gdev = self.device if on_gpu else "cpu"

        def gen(sub):
            g = torch.Generator(device=gdev)
            g.manual_seed(seed * 100003 + sub)
            return g

        def rn(g, *shape, std=1.0):
            return (torch.randn(*shape, generator=g, device=gdev)
                    * std).to(torch.bfloat16)

        def ru(g, n, lo, hi):
            return (torch.rand(n, generator=g, device=gdev)
                    * (hi - lo) + lo).to(torch.bfloat16)

        for lid in self.layer_ids:
            g = gen(lid)
            nq, nkv, d, dv = self._dims(lid)
            ff = self._ff(lid)
            t = {
                "norm1": 1 + rn(g, W, std=0.1),
                "mix.q": rn(g, nq * d, W, std=W ** -0.5),
                "mix.k": rn(g, nkv * d, W, std=W ** -0.5),
                "mix.v": rn(g, nkv * dv, W, std=W ** -0.5),
                "mix.q.norm": 1 + rn(g, nq * d, std=0.1),
                "mix.k.norm": 1 + rn(g, nkv * d, std=0.1),
                "mix.temp": ru(g, nq, 0.5, 2.0),
                "mix.r1": ru(g, nq, 0.0, 1.0),
                "mix.r2": ru(g, nq, 0.05, 1.0),
                "mix.sink": rn(g, nq),
                "mix.o": rn(g, W, nq * dv, std=(nq * dv) ** -0.5),
                "ls1": ru(g, W, 0.2, 1.0),
            }
            if ff:
                t["mlp.up"] = rn(g, ff, W, std=W ** -0.5)
                t["mlp.down"] = rn(g, W, ff, std=ff ** -0.5)
                t["mlp.act"] = rn(g, 2, std=0.5)
                t["ls2"] = ru(g, W, 0.2, 1.0)
            self.layers[lid] = self._build_layer(lid, t.__getitem__)
        if self.is_first:
            self.embed = rn(gen(99991), c.vocab_size, W).to(
                self.wdtype).to(self.device)
        if self.is_last:
            self.final_norm = self._vec(1 + rn(gen(99993), W, std=0.1))
            self.lm_head = self._lin(rn(gen(99992), c.vocab_size, W,
                                        std=W ** -0.5))

    # ---------- forward ----------

    def embed_tokens(self, tokens: torch.Tensor) -> torch.Tensor:
        assert self.embed is not None, "this shard does not own the embedding"
        e = torch.nn.functional.embedding(tokens, self.embed)
        return e.to(torch.float32) * self.cfg.embedding_scale

    def _window(self, x: torch.Tensor, layer_ids: Sequence[int], kv: KVCache,
                pos: torch.Tensor, T: int, lens, slots) -> None:
        """Run the layers of one window over x [B*T, W] fp32 (in place).
        Token (b, t) sits at position pos[b]+t of cache row slots[b]."""
        c = self.cfg
        eps = c.rms_eps
        wdt = self.wdtype
        u = None
        layer_ids = list(layer_ids)
        for i, lid in enumerate(layer_ids):
            lw = self._layer(lid)
            nq, nkv, d, dv = self._dims(lid)
            m = c.layer_specs[lid]["mixer"]
            if u is None:
                u = ops.rmsnorm_rows(x, lw.attn_norm, eps, wdt)
            li = kv.local[lid]
            qkv = lw.qkv(u)
            q = ops.qknorm_append(qkv, lw.q_norm, lw.k_norm, eps, nq, nkv, d,
                                  dv, kv.k[li], kv.v[li], pos, T, lens,
                                  slots)
            a = ops.attn_mod(q, kv.k[li], kv.v[li], pos, T,
                             float(m["scale"]), lens, slots, temp=lw.temp,
                             softcap=float(m.get("softcap") or 0.0),
                             dist_r1=lw.dist_r1, dist_r2=lw.dist_r2,
                             sinks=lw.sinks)
            o = lw.o(a)
            f = None
            if lw.up is not None:
                f = lw.down(ops.xielu(lw.up(u), lw.act_pq))
            # residual update fused with the next layer's norm (resident
            # layers only: binding the next layer of a streamed window here
            # could recycle the slot this layer's scales still live in)
            nxt = (self.layers[layer_ids[i + 1]].attn_norm
                   if i + 1 < len(layer_ids)
                   and layer_ids[i + 1] in self.layers else None)
            u = ops.ls_resid_rmsnorm(x, o, lw.ls1, f, lw.ls2, nxt, eps, wdt)
            if self._obs_sync:
                self._profile_layer_sync(lid)

    def decode_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                      kv: KVCache) -> torch.Tensor:
        """One decode step. h [B, W] fp32, modified in place; kv.pos holds
        each row's write position."""
        if layer_ids:
            self._window(h, layer_ids, kv, kv.pos, 1, None, None)
        return h

    def prefill_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                       kv: KVCache, p0, lens: Optional[torch.Tensor] = None,
                       slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Prefill h [B, T, W] fp32 in place. ``p0``: first position, an
        int (every row) or an int32 tensor [B]. ``lens`` [B] int32: real
        token count per row (rows are right-padded to T; padding is never
        appended to the cache and its outputs are meaningless). ``slots``
        [B] int32: cache row of each batch row (default: row b)."""
        if not layer_ids:
            return h
        B, T, W = h.shape
        if not torch.is_tensor(p0):
            p0 = torch.full((B,), int(p0), dtype=torch.int32,
                            device=h.device)
        self._window(h.view(B * T, W), layer_ids, kv, p0, T, lens, slots)
        return h

    def normalize_project(self, h: torch.Tensor) -> torch.Tensor:
        assert self.final_norm is not None and self.lm_head is not None
        y = ops.rmsnorm_rows(h, self.final_norm, self.cfg.rms_eps,
                             self.wdtype)
        return self.lm_head(y)
