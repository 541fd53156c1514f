"""Gegorax ring model: heterogeneous sequence-state layers on an fp32 residual.

Every layer normalizes the residual once and feeds a mixer and a feed-forward
from the same normalized activations; afterwards a per-layer token input is
added:

    u = rmsnorm(x) * g
    x <- x + mixer(u) + ff(u)                              (x kept in fp32)
    x <- x + rms(P_s (gelu_tanh(G_s x) * e_l[token])) * s  (optional)

with e_l[token] the layer's slice of a second embedding row of the token.

Mixers (``cfg.layer_specs[l]["type"]``):

* ``parallel``: two mixers read the same u and their outputs, each
  RMS-normalized over the model width with its own weight, are averaged.
  Left: grouped-head attention with per-head q/k norm, an interleaved partial
  rotation, a sliding window, and beside the window one pooled key/value (the
  block mean of the cache) per whole block of positions before it. Right: a
  selective state-space layer with a scalar decay per head (short causal
  convolution, softplus step size, gate before a grouped norm).
* ``general_delta``: a generalized delta rule, per head
  S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r, with a low-rank decay
  projection, per-head output norm and a sigmoid output gate.

Feed-forwards: dense (up -> relu^2 -> down) or a mixture of clamped-GLU
experts (top-k by router logit, softmax over the chosen logits, optional
always-on shared expert).

Per-slot sequence state lives in the framework's cache object
(``KVCache.state``): keys/values plus pooled-block caches for attention,
convolution tails and fp32 recurrent states for the others. All state is
taken as zero at position 0 and is never touched by padding or idle rows, so
slots are reused without a reset and a ragged batch equals each row alone.

Checkpoint names: ``embed``, ``side.embed``, ``l<i>.norm1``,
``l<i>.mix.left.{q,k,v,o,q.norm,k.norm,out}``,
``l<i>.mix.right.{in,conv,conv.b,dt_bias,A_log,D,norm,o,out}``,
``l<i>.mix.{r,k,v,g,a,a.b,w1,w2,w0,norm,o}``, ``l<i>.mlp.{up,down}``,
``l<i>.mlp.{router,router.b,e<j>.{gate,up,down},shared.{gate,up,down}}``,
``l<i>.side.{gate,proj,norm}``, ``final.norm``, ``head``.

``cfg.compute_dtype == "float32"`` runs weights, activations, caches and every
product in true fp32.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch

from .. import ops
from .base import KVCache, LayerWeights, Linear, RingModel
from .config import ModelConfig
from .moe import stack_experts

GLU_ALPHA = 1.702               # sigmoid slope of the experts' gate
DELTA_DECAY_SCALE = math.exp(-0.5)
DELTA_UNIT_EPS = 1e-6


class GegoraxRingModel(RingModel):
    model_type = "gegorax"
    model_types = ["gegorax"]
    act_dtype = torch.float32          # residual stream / ring hops
    ragged_prefill = True
    supports_float32 = True
    # layers read the token ids again: the executor calls set_tokens on
    # every pipeline stage
    needs_tokens = True
    stateful = True                    # idle decode rows must not step
    supports_offload = False           # layer kinds hold different tensors
    DENSE_MOE_MAX_T = 64

    def __init__(self, cfg: ModelConfig, layer_ids: Sequence[int], device,
                 is_first: bool, is_last: bool, smax: int = 4096, **kw):
        if kw.get("tp_size", 1) > 1 or kw.get("cp_size", 1) > 1:
            raise NotImplementedError(
                "gegorax: tensor/context parallelism inside a stage is not "
                "implemented")
        assert cfg.layer_specs is not None, "gegorax needs per-layer specs"
        assert cfg.quant is None, "gegorax: bf16 / fp32 weights only"
        super().__init__(cfg, layer_ids, device, is_first, is_last,
                         smax=smax, **kw)
        self.wdtype = (torch.float32 if cfg.compute_dtype == "float32"
                       else torch.bfloat16)
        self.logits_dtype = self.wdtype
        self.side_embed: Optional[torch.Tensor] = None
        self._tokens: Optional[torch.Tensor] = None

    def _init_positional(self):
        pass        # angles are computed from positions inside the kernel

    # ---------- per-layer sizes ----------

    def _spec(self, lid: int) -> dict:
        return self.cfg.layer_specs[lid]

    def _ssm_dims(self, m: dict):
        heads, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
        return heads, P, N, G, heads * P, heads * P + 2 * G * N

    def make_kv_cache(self, batch: int, smax: int) -> KVCache:
        dims, states = [], []
        for lid in self.layer_ids:
            s = self._spec(lid)
            m = s["mixer"]
            if s["type"] == "parallel":
                lf, rt = m["left"], m["right"]
                heads, P, N, G, inner, C = self._ssm_dims(rt)
                dims.append((lf["kv_heads"], lf["dim"], lf["vdim"]))
                st = {"conv": ((max(int(rt["conv"]) - 1, 0), C), self.wdtype),
                      "ssm": ((heads, N, P), torch.float32)}
                pool = int((lf.get("mask") or {}).get("pool") or 0)
                if pool:
                    nb = smax // pool + 1
                    st["pk"] = ((lf["kv_heads"], nb, lf["dim"]), self.wdtype)
                    st["pv"] = ((lf["kv_heads"], nb, lf["vdim"]), self.wdtype)
                states.append(st)
            else:
                dims.append(None)
                states.append({"S": ((m["heads"], m["dim"], m["dim"]),
                                     torch.float32)})
        return KVCache(self.cfg, self.layer_ids, batch, smax, self.device,
                       layer_dims=dims, dtype=self.wdtype,
                       layer_state=states)

    # ---------- weights ----------

    def _lin(self, w: torch.Tensor, bias=None) -> Linear:
        return Linear(w.to(self.wdtype).to(self.device).contiguous(), bias)

    def _vec(self, t: torch.Tensor) -> torch.Tensor:
        # small per-channel / per-head parameters feed fp32 math directly
        return t.to(torch.float32).to(self.device).contiguous()

    def _build_layer(self, lid: int, get) -> LayerWeights:
        s = self._spec(lid)
        m = s["mixer"]
        W = self.cfg.hidden_size
        lw = LayerWeights(attn_norm=self._vec(get("norm1")))
        if s["type"] == "parallel":
            lf, rt = m["left"], m["right"]
            H, G, d, dv = lf["heads"], lf["kv_heads"], lf["dim"], lf["vdim"]
            q, k, v = (get("mix.left." + n) for n in "qkv")
            assert q.shape == (H * d, W) and k.shape == (G * d, W) \
                and v.shape == (G * dv, W), f"layer {lid}: attention shapes"
            lw.qkv = self._lin(torch.cat([q, k, v]))
            lw.q_norm = self._vec(get("mix.left.q.norm"))
            lw.k_norm = self._vec(get("mix.left.k.norm"))
            lw.o = self._lin(get("mix.left.o"))
            rot = lf.get("rot")
            lw.rot_freq = None
            if rot and int(rot["dims"]) >= 2:
                n = int(rot["dims"])
                assert n % 2 == 0 and n <= d, f"layer {lid}: rot.dims"
                f = [float(rot["base"]) ** (-2.0 * i / n)
                     for i in range(n // 2)]
                lw.rot_freq = torch.tensor(f, dtype=torch.float32,
                                           device=self.device)
            heads, P, N, Gs, inner, C = self._ssm_dims(rt)
            win = get("mix.right.in")
            assert win.shape == (2 * inner + 2 * Gs * N + heads, W), \
                f"layer {lid}: state-space projection shape"
            lw.ssm_in = self._lin(win)
            lw.conv_w = self._vec(get("mix.right.conv"))
            assert lw.conv_w.shape == (C, int(rt["conv"]))
            lw.conv_b = self._vec(get("mix.right.conv.b"))
            lw.dt_bias = self._vec(get("mix.right.dt_bias"))
            lw.a_log = self._vec(get("mix.right.A_log"))
            lw.dskip = self._vec(get("mix.right.D"))
            lw.ssm_norm = self._vec(get("mix.right.norm"))
            lw.ssm_o = self._lin(get("mix.right.o"))
            lw.left_out = self._vec(get("mix.left.out"))
            lw.right_out = self._vec(get("mix.right.out"))
        else:
            H, d = m["heads"], m["dim"]
            parts = [get("mix." + n) for n in ("r", "k", "v", "g", "a", "w1")]
            assert all(p.shape == (H * d, W) for p in parts[:5]), \
                f"layer {lid}: delta-rule shapes"
            lw.qkv = self._lin(torch.cat(parts))        # [r;k;v;g;a;w1]
            lw.w2 = self._lin(get("mix.w2"))
            lw.w0 = self._vec(get("mix.w0"))
            lw.a_b = self._vec(get("mix.a.b"))
            lw.delta_norm = self._vec(get("mix.norm"))
            lw.o = self._lin(get("mix.o"))
        ff = s.get("mlp")
        lw.up = None
        if ff is not None and ff["kind"] == "dense":
            lw.up = self._lin(get("mlp.up"))
            lw.down = self._lin(get("mlp.down"))
        elif ff is not None:
            E = int(ff["router"]["experts"])
            # the router runs in fp32 whatever the activation dtype
            lw.router = Linear(self._vec(get("mlp.router")),
                               self._vec(get("mlp.router.b")))
            lw.experts_gateup = [
                self._lin(torch.cat([get(f"mlp.e{e}.gate"),
                                     get(f"mlp.e{e}.up")])) for e in range(E)]
            lw.experts_down = [self._lin(get(f"mlp.e{e}.down"))
                               for e in range(E)]
            if ff.get("shared"):
                lw.shared_gateup = self._lin(torch.cat(
                    [get("mlp.shared.gate"), get("mlp.shared.up")]))
                lw.shared_down = self._lin(get("mlp.shared.down"))
        if self.cfg.token_side_dim:
            lw.side_gate = self._lin(get("side.gate"))
            lw.side_proj = self._lin(get("side.proj"))
            lw.side_norm = self._vec(get("side.norm"))
        return lw

    def load_state_dict(self, sd: dict):
        for lid in self.layer_ids:
            self.layers[lid] = self._build_layer(
                lid, lambda n, p=f"l{lid}.": sd[p + n])
        if self.cfg.token_side_dim and self.layer_ids:
            self.side_embed = sd["side.embed"].to(self.wdtype).to(
                self.device).contiguous()
        if self.is_first:
            self.embed = sd["embed"].to(self.wdtype).to(self.device)
        if self.is_last:
            self.final_norm = self._vec(sd["final.norm"])
            self.lm_head = self._lin(sd["head"])

    def init_random(self, seed: int = 0):
        """Seeded per layer id (any sharding of one (model, seed) holds the
        same global weights); scales keep every branch of comparable size."""
        c = self.cfg
        W = c.hidden_size
        gdev = self.device if self.device.type == "cuda" else "cpu"

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

        def lin(g, out, inp):
            return rn(g, out, inp, std=inp ** -0.5)

        sd = c.token_side_dim
        for lid in self.layer_ids:
            g = gen(lid)
            s = self._spec(lid)
            m = s["mixer"]
            t = {"norm1": 1 + rn(g, W, std=0.1)}
            if s["type"] == "parallel":
                lf, rt = m["left"], m["right"]
                H, G, d, dv = lf["heads"], lf["kv_heads"], lf["dim"], lf["vdim"]
                heads, P, N, Gs, inner, C = self._ssm_dims(rt)
                t.update({
                    "mix.left.q": lin(g, H * d, W),
                    "mix.left.k": lin(g, G * d, W),
                    "mix.left.v": lin(g, G * dv, W),
                    "mix.left.q.norm": 1 + rn(g, d, std=0.1),
                    "mix.left.k.norm": 1 + rn(g, d, std=0.1),
                    "mix.left.o": lin(g, W, H * dv),
                    "mix.right.in": lin(g, 2 * inner + 2 * Gs * N + heads, W),
                    "mix.right.conv": rn(g, C, int(rt["conv"]), std=0.5),
                    "mix.right.conv.b": rn(g, C, std=0.1),
                    "mix.right.dt_bias": ru(g, heads, -3.0, 0.0),
                    "mix.right.A_log": ru(g, heads, -1.0, 1.5),
                    "mix.right.D": rn(g, heads),
                    "mix.right.norm": 1 + rn(g, inner, std=0.1),
                    "mix.right.o": lin(g, W, inner),
                    "mix.left.out": 1 + rn(g, W, std=0.1),
                    "mix.right.out": 1 + rn(g, W, std=0.1)})
            else:
                H, d = m["heads"], m["dim"]
                rank = max(8, (H * d) // 16)
                for n in ("r", "k", "v", "g", "a"):
                    t["mix." + n] = lin(g, H * d, W)
                t.update({"mix.a.b": rn(g, H * d, std=0.5),
                          "mix.w1": lin(g, rank, W),
                          "mix.w2": lin(g, H * d, rank),
                          "mix.w0": rn(g, H * d),
                          "mix.norm": 1 + rn(g, H * d, std=0.1),
                          "mix.o": lin(g, W, H * d)})
            ff = s.get("mlp")
            if ff is not None and ff["kind"] == "dense":
                t["mlp.up"] = lin(g, ff["ff"], W)
                t["mlp.down"] = lin(g, W, ff["ff"])
            elif ff is not None:
                ef = ff["expert"]["ff"]
                t["mlp.router"] = lin(g, ff["router"]["experts"], W)
                t["mlp.router.b"] = rn(g, ff["router"]["experts"], std=0.1)
                names = [f"e{e}" for e in range(ff["router"]["experts"])]
                sizes = [ef] * len(names)
                if ff.get("shared"):
                    names.append("shared")
                    sizes.append(ff["shared"]["ff"])
                for n, sz in zip(names, sizes):
                    t[f"mlp.{n}.gate"] = lin(g, sz, W)
                    t[f"mlp.{n}.up"] = lin(g, sz, W)
                    t[f"mlp.{n}.down"] = lin(g, W, sz)
            if sd:
                t["side.gate"] = lin(g, sd, W)
                t["side.proj"] = lin(g, W, sd)
                t["side.norm"] = ru(g, W, 0.2, 1.0)
            self.layers[lid] = self._build_layer(lid, t.__getitem__)
        if sd and self.layer_ids:
            self.side_embed = rn(gen(99994), c.vocab_size,
                                 sd * c.num_layers).to(self.wdtype).to(
                                     self.device)
        if self.is_first:
            self.embed = rn(gen(99991), c.vocab_size, W).to(
                self.wdtype).to(self.device)
        if self.is_last:
            self.final_norm = self._vec(1 + rn(gen(99993), W, std=0.1))
            self.lm_head = self._lin(lin(gen(99992), c.vocab_size, W))

    # ---------- forward ----------

    def set_tokens(self, tokens: torch.Tensor) -> None:
        """Token ids of the rows the next window call runs ([B] or [B, T],
        on this model's device): the per-layer token input reads them."""
        self._tokens = tokens

    def embed_tokens(self, tokens: torch.Tensor) -> torch.Tensor:
        assert self.embed is not None, "this shard does not own the embedding"
        self.set_tokens(tokens)
        return torch.nn.functional.embedding(tokens, self.embed).to(
            torch.float32)

    def _attention(self, u, lw, m, kv, li, pos, T, lens, slots):
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        mask = m.get("mask") or {}
        size, pool = int(mask.get("size") or 0), int(mask.get("pool") or 0)
        q = ops.qknorm_append(lw.qkv(u), lw.q_norm, lw.k_norm,
                              self.cfg.rms_eps, H, G, d, dv, kv.k[li],
                              kv.v[li], pos, T, lens, slots, per_head=True,
                              rot_freq=lw.rot_freq)
        st = kv.state[li]
        if pool:
            ops.kv_pool_update(kv.k[li], kv.v[li], st["pk"], st["pv"], pos,
                               T, pool, lens, slots)
        a = ops.attn_mod(q, kv.k[li], kv.v[li], pos, T, float(m["scale"]),
                         lens, slots, window=size,
                         pool_k=st.get("pk"), pool_v=st.get("pv"), pool=pool)
        return lw.o(a)

    def _ssd(self, u, lw, m, kv, li, pos, T, lens, slots):
        heads, P, N, G, inner, C = self._ssm_dims(m)
        st = kv.state[li]
        zx = lw.ssm_in(u)                      # [z | x B C | dt]
        xbc = ops.causal_conv_silu(zx, inner, lw.conv_w, lw.conv_b,
                                   st["conv"], pos, T, lens, slots)
        y = ops.ssd_scan(xbc, zx, inner + C, lw.dt_bias, lw.a_log, lw.dskip,
                         st["ssm"], pos, T, heads, P, N, G, lens, slots)
        yg = ops.gated_group_rmsnorm(y, zx, 0, lw.ssm_norm,
                                     int(m["norm_groups"]), self.cfg.rms_eps,
                                     "silu", True, self.wdtype)
        return lw.ssm_o(yg)

    def _delta(self, u, lw, m, kv, li, pos, T, lens, slots):
        H, d = m["heads"], m["dim"]
        n = H * d
        p = lw.qkv(u)                          # [r | k | v | g | a | w1]
        wl = lw.w2(ops.act_slice(p, 5 * n, p.shape[1] - 5 * n, "tanh"))
        o = ops.delta_scan(p, 0, n, 2 * n, 4 * n, wl, lw.w0, lw.a_b,
                           kv.state[li]["S"], pos, T, H, d,
                           DELTA_DECAY_SCALE, DELTA_UNIT_EPS, lens, slots)
        og = ops.gated_group_rmsnorm(o, p, 3 * n, lw.delta_norm, H,
                                     self.cfg.rms_eps, "sigmoid", False,
                                     self.wdtype)
        return lw.o(og)

    def _expert(self, x, gateup: Linear, down: Linear, limit: float):
        return down(ops.clamped_glu(gateup(x), GLU_ALPHA, limit))

    def _moe(self, u, lw, ff):
        c = self.cfg
        T = u.shape[0]
        E, top = int(ff["router"]["experts"]), int(ff["router"]["top"])
        limit = float(ff["expert"]["limit"])
        logits = lw.router(u.float())
        val, idx = torch.topk(logits, top, dim=-1)
        we = torch.zeros(T, E, dtype=torch.float32, device=u.device)
        we.scatter_(1, idx, torch.softmax(val, dim=-1))
        eg0 = lw.experts_gateup[0]
        if (T <= self.DENSE_MOE_MAX_T and self.wdtype == torch.bfloat16
                and eg0.in_features % 8 == 0
                and (eg0.out_features // 2) % 8 == 0):
            # grouped expert kernels: two launches, unrouted experts skipped
            # on the device (no host sync: graph-capturable)
            st = stack_experts(lw, list(range(E)))
            act = ops.moe_gateup(u, st["gw"], None, None, we, 0, False, 1,
                                 GLU_ALPHA, limit)
            out = ops.moe_down(act, st["dw"], None, None, we, 0, False)
        elif T <= self.DENSE_MOE_MAX_T:
            # few rows: every expert on every row, weighted (zero for the
            # experts a row did not choose); no host sync
            out = torch.zeros(T, c.hidden_size, dtype=torch.float32,
                              device=u.device)
            for e in range(E):
                out += we[:, e:e + 1] * self._expert(
                    u, lw.experts_gateup[e], lw.experts_down[e],
                    limit).float()
        else:
            out = torch.zeros(T, c.hidden_size, dtype=torch.float32,
                              device=u.device)
            hit = (we > 0).any(dim=0).tolist()
            for e in range(E):
                if not hit[e]:
                    continue
                rows = (we[:, e] > 0).nonzero(as_tuple=True)[0]
                d = self._expert(u[rows].contiguous(), lw.experts_gateup[e],
                                 lw.experts_down[e], limit)
                out.index_add_(0, rows, d.float() * we[rows, e:e + 1])
        if getattr(lw, "shared_gateup", None) is not None:
            out = out + self._expert(u, lw.shared_gateup, lw.shared_down,
                                     float(ff["shared"]["limit"])).float()
        return out

    def _ff(self, u, lw, ff):
        if ff is None:
            return None
        if ff["kind"] == "dense":
            z = lw.up(u)
            return lw.down(ops.act_slice(z, 0, z.shape[1], "relu_sq"))
        return self._moe(u, lw, ff)

    def _window(self, x: torch.Tensor, layer_ids: Sequence[int], kv: KVCache,
                pos: torch.Tensor, T: int, lens, slots) -> None:
        """Run the layers of one window over x [B*T, W] fp32 (in place).
        Token (b, t) sits at position pos[b]+t of cache row slots[b]."""
        c = self.cfg
        eps, wdt, side = c.rms_eps, self.wdtype, c.token_side_dim
        cast = wdt != torch.float32
        tokens = None
        if side:
            assert self._tokens is not None and \
                self._tokens.numel() == x.shape[0], \
                "gegorax: the window needs this step's token ids"
            tokens = self._tokens.reshape(-1)
        u = None
        layer_ids = list(layer_ids)
        for i, lid in enumerate(layer_ids):
            lw = self._layer(lid)
            s = self._spec(lid)
            li = kv.local[lid]
            if u is None:
                u = ops.rmsnorm_rows(x, lw.attn_norm, eps, wdt)
            if s["type"] == "parallel":
                a = self._attention(u, lw, s["mixer"]["left"], kv, li, pos,
                                    T, lens, slots)
                b = self._ssd(u, lw, s["mixer"]["right"], kv, li, pos, T,
                              lens, slots)
                wa, wb, coef = lw.left_out, lw.right_out, 0.5
            else:
                a = self._delta(u, lw, s["mixer"], kv, li, pos, T, lens,
                                slots)
                b = wa = wb = None
                coef = 1.0
            f = self._ff(u, lw, s.get("mlp"))
            nxt = (self.layers[layer_ids[i + 1]].attn_norm
                   if i + 1 < len(layer_ids)
                   and layer_ids[i + 1] in self.layers else None)
            if side:
                _, xc = ops.resid_branches_rmsnorm(
                    x, a, wa, b, wb, coef, f, None, eps, wdt, want_cast=cast)
                g = ops.gelu_gather_mul(lw.side_gate(xc if cast else x),
                                        self.side_embed, tokens, lid * side)
                u, _ = ops.resid_branches_rmsnorm(
                    x, lw.side_proj(g), lw.side_norm, None, None, 1.0, None,
                    nxt, eps, wdt)
            else:
                u, _ = ops.resid_branches_rmsnorm(
                    x, a, wa, b, wb, coef, f, nxt, eps, wdt)
            if self._obs_sync:
                self._profile_layer_sync(lid)

    def decode_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                      kv: KVCache) -> torch.Tensor:
        """One decode step. h [B, W] fp32, modified in place; kv.pos holds
        each row's write position; rows flagged in kv.idle keep their state
        (they run as padding)."""
        if layer_ids:
            self._window(h, layer_ids, kv, kv.pos, 1,
                         (~kv.idle).to(torch.int32), None)
        return h

    def prefill_window(self, h: torch.Tensor, layer_ids: Sequence[int],
                       kv: KVCache, p0, lens: Optional[torch.Tensor] = None,
                       slots: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Prefill h [B, T, W] fp32 in place. ``p0``: first position, an int
        (every row) or an int32 tensor [B]. ``lens`` [B] int32: real token
        count per row (rows are right-padded to T; padding never reaches the
        cache or any state and its outputs are meaningless). ``slots`` [B]
        int32: cache row of each batch row (default: row b)."""
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

    def weight_bytes(self) -> int:
        """Bytes of every tensor and linear the resident layers hold (the
        layer kinds carry different sets of them)."""
        def size(v) -> int:
            if isinstance(v, Linear):
                return v.nbytes()
            if torch.is_tensor(v):
                return v.numel() * v.element_size()
            if isinstance(v, (list, tuple)):
                return sum(size(x) for x in v)
            return 0
        return sum(size(v) for lw in self.layers.values()
                   for k, v in vars(lw).items() if k != "experts_stacked")
