"""Posudra in the framework against the plain oracle (tests/posudra_oracle.py).

Every test builds its own small configuration and random checkpoint, loads
it through the framework's model / cache / executor (and, for generation,
the shard runtime's slot scheduler) and compares logits with the oracle,
which is written from the equations and shares no code with dnet_amd.
Model-level tests run on the CPU reference-op path and, marked ``gpu``, on
the HIP kernels.
"""
import io
import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import posudra_oracle as O
from dnet_amd.models import ModelConfig, get_ring_model
from dnet_amd.parallel.ring import RingExecutor

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


# ---------- small random checkpoints ----------

def mixer(heads, kv, dim, vdim, scale=0.3, softcap=4.0):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim,
         "scale": scale}
    if softcap is not None:
        m["softcap"] = softcap
    return m


def make_cfg(layers, width=48, vocab=97, eps=1e-5, emb=3.0):
    return {"architecture": "Posudra", "vocab": vocab, "width": width,
            "norm": {"eps": eps}, "embedding": {"scale": emb},
            "layers": [{"type": "attention", "mixer": m,
                        "mlp": None if ff is None else
                        {"kind": "dense", "ff": ff}} for m, ff in layers]}


def make_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rn(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

    def ru(n, lo, hi):
        return (torch.rand(n, generator=g) * (hi - lo) + lo).to(torch.bfloat16)

    sd = {"embed": rn(V, W), "final.norm": 1 + rn(W, std=0.2),
          "head": rn(V, W, std=W ** -0.5)}
    for i, spec in enumerate(cfg["layers"]):
        m = spec["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        p = f"l{i}."
        sd.update({
            p + "norm1": 1 + rn(W, std=0.2),
            p + "mix.q": rn(H * d, W, std=W ** -0.5),
            p + "mix.k": rn(G * d, W, std=W ** -0.5),
            p + "mix.v": rn(G * dv, W, std=W ** -0.5),
            p + "mix.q.norm": 1 + rn(H * d, std=0.3),
            p + "mix.k.norm": 1 + rn(G * d, std=0.3),
            p + "mix.temp": ru(H, 0.5, 3.0),
            p + "mix.r1": ru(H, 0.0, 1.5),
            p + "mix.r2": ru(H, 0.05, 2.0),
            p + "mix.sink": rn(H, std=2.0),
            p + "mix.o": rn(W, H * dv, std=(H * dv) ** -0.5),
            p + "ls1": ru(W, 0.2, 1.2),
        })
        if spec["mlp"] is not None:
            ff = spec["mlp"]["ff"]
            sd.update({p + "mlp.up": rn(ff, W, std=2 * W ** -0.5),
                       p + "mlp.down": rn(W, ff, std=ff ** -0.5),
                       p + "mlp.act": rn(2, std=1.0),
                       p + "ls2": ru(W, 0.2, 1.2)})
    return sd


BASE = [(mixer(4, 2, 16, 8), 40), (mixer(6, 2, 8, 24, scale=0.5), None),
        (mixer(2, 2, 20, 12, softcap=None), 72),
        (mixer(3, 1, 16, 16, scale=1.0, softcap=1.5), 24)]


def executor(cfg, sd, device, dtype="float32", slots=4, smax=320, **kw):
    mc = ModelConfig.from_hf(cfg)
    mc.compute_dtype = dtype
    ex = RingExecutor(mc, 0, 1, device, mb_size=slots, smax=smax,
                      init_weights=False, use_graphs=kw.pop("graphs", False),
                      **kw)
    ex.model.load_state_dict(sd)
    return ex


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g)


def close(got, want, dtype="float32"):
    want = want.to(torch.float32)
    scale = float(want.pow(2).mean().sqrt())
    tol = 3e-4 if dtype == "float32" else 6e-2
    err = float((got.float().cpu() - want).abs().max())
    assert err <= tol * scale, f"max err {err:.3e} vs rms {scale:.3e}"


def decode_steps(ex, slot_tokens, park=None):
    """One slot-batch decode step feeding the given token per live slot;
    returns the logits buffer [slots, V] (fp32)."""
    tb = ex.tokbuf[0].cpu()
    live = torch.zeros(ex.mb_size, dtype=torch.bool)
    for s, t in slot_tokens.items():
        tb[s] = int(t)
        live[s] = True
    ex.tokbuf[0].copy_(tb)
    ex.slot_step_compute()
    lg = ex.logits_buf[0].float().cpu().clone()
    dead = (~live).to(ex.device)
    ex.slot_advance(dead, dead)
    return lg


# ---------- configuration and registry ----------

def test_config_and_registry():
    cfg = make_cfg(BASE)
    mc = ModelConfig.from_hf(cfg)
    assert mc.model_type == "posudra" and mc.num_layers == 4
    assert mc.hidden_size == 48 and mc.vocab_size == 97
    assert mc.layer_specs[1]["mlp"] is None
    assert get_ring_model("posudra").__name__ == "PosudraRingModel"
    bad = make_cfg(BASE)
    bad["layers"][0]["type"] = "recurrent"
    with pytest.raises(ValueError):
        ModelConfig.from_hf(bad)
    ex = executor(cfg, make_weights(cfg), "cpu", slots=2, smax=16)
    kv = ex.kvs[0]
    assert [tuple(t.shape) for t in kv.k] == [
        (2, 2, 16, 16), (2, 2, 16, 8), (2, 2, 16, 20), (2, 1, 16, 16)]
    assert [t.shape[-1] for t in kv.v] == [8, 24, 12, 16]
    assert ex.hbuf[0].dtype == torch.float32      # fp32 residual stream


# ---------- each mechanism alone (ops vs oracle) ----------

@pytest.mark.parametrize("device", DEVICES)
def test_xielu_both_branches(device):
    import dnet_amd.ops as ops
    z = torch.tensor([[-30.0, -3.0, -1e-3, 0.0, 1e-3, 0.5, 7.0]])
    for p, q in ((0.4, -0.6), (-3.0, 2.0), (0.0, 0.0)):
        pq = torch.tensor([p, q])
        got = ops.xielu(z.to(device), pq.to(device)).cpu()
        want = O.xielu(z.double(), pq[0].double(), pq[1].double())
        torch.testing.assert_close(got.double(), want, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_norm_whole_projection_vs_per_head(device):
    """The q/k norm runs over ALL heads at once: one head scaled up must
    shrink the others (a per-head norm would not)."""
    import dnet_amd.ops as ops
    H, G, d, dv = 3, 1, 8, 4
    qkv = torch.randn(1, (H + G) * d + G * dv)
    qkv[0, :d] *= 50.0                                  # head 0 dominates
    qw, kw = torch.rand(H * d) + 0.5, torch.rand(G * d) + 0.5
    kc, vc = torch.zeros(1, G, 4, d), torch.zeros(1, G, 4, dv)
    pos = torch.zeros(1, dtype=torch.int32)
    q = ops.qknorm_append(qkv.to(device), qw.to(device), kw.to(device), 1e-6,
                          H, G, d, dv, kc.to(device), vc.to(device),
                          pos.to(device), 1).cpu()
    want = O.rms(qkv[:, :H * d].double(), 1e-6) * qw.double()
    torch.testing.assert_close(q.double(), want, atol=1e-5, rtol=1e-5)
    assert float(q[0, d:].abs().max()) < 0.2            # others squeezed


def _attn_case(device, T, H, G, d, dv, w, q, k, v, mx):
    """Run the framework ops on given per-position q/k/v (already normed)
    and return [T, H*dv]."""
    import dnet_amd.ops as ops
    smax = T + 3
    kc = torch.zeros(1, G, smax, d)
    vc = torch.zeros(1, G, smax, dv)
    kc[0, :, :T] = k.view(T, G, d).transpose(0, 1)
    vc[0, :, :T] = v.view(T, G, dv).transpose(0, 1)
    f = lambda n: w[n].float().to(device)
    out = ops.attn_mod(q.float().to(device), kc.to(device), vc.to(device),
                       torch.zeros(1, dtype=torch.int32, device=device), T,
                       mx["scale"], temp=f("mix.temp"),
                       softcap=mx.get("softcap") or 0.0,
                       dist_r1=f("mix.r1"), dist_r2=f("mix.r2"),
                       sinks=f("mix.sink"))
    return out.cpu()


def _oracle_attn(T, H, G, d, dv, w, q, k, v, mx):
    outs = []
    for h in range(H):
        g = h // (H // G)
        s = O.attention_scores(q.view(T, H, d)[:, h].double(),
                               k.view(T, G, d)[:, g].double(), h, mx, w)
        p = O.sink_softmax(s, w["mix.sink"][h])
        outs.append(p @ v.view(T, G, dv)[:, g].double())
    return torch.cat(outs, dim=-1)


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds(device):
    """One key 500 positions back is made to stand out (its query match is
    scaled up): losing it, or mis-measuring its distance, shows."""
    T, H, G, d, dv = 600, 2, 1, 16, 8
    torch.manual_seed(5)
    q, k = torch.randn(T, H * d) * 0.3, torch.randn(T, G * d) * 0.3
    v = torch.randn(T, G * dv)
    far, at = 77, 577
    k[far] = 0.0
    k[far, :4] = 4.0
    q[at, :4] = 4.0
    q[at, d:d + 4] = 4.0
    w = {"mix.temp": torch.tensor([1.0, 2.0]).double(),
         "mix.r1": torch.tensor([0.7, 0.2]).double(),
         "mix.r2": torch.tensor([0.5, 1.0]).double(),
         "mix.sink": torch.tensor([0.5, -1.0]).double()}
    mx = {"scale": 0.5, "softcap": 30.0}
    want = _oracle_attn(T, H, G, d, dv, w, q, k, v, mx)
    s = O.attention_scores(q.view(T, H, d)[:, 0].double(), k.double(), 0, mx, w)
    assert float(O.sink_softmax(s, w["mix.sink"][0])[at, far]) > 0.5
    got = _attn_case(device, T, H, G, d, dv, w, q, k, v, mx)
    torch.testing.assert_close(got.double(), want, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_sink_cap_and_distance_each_matter(device):
    """Scores large enough that the cap bites, a sink that takes most of
    the mass on one head, a distance penalty that reorders keys."""
    T, H, G, d, dv = 70, 2, 2, 8, 8
    torch.manual_seed(6)
    q, k = torch.randn(T, H * d) * 3, torch.randn(T, G * d) * 3
    v = torch.randn(T, G * dv)
    w = {"mix.temp": torch.tensor([2.5, 0.5]).double(),
         "mix.r1": torch.tensor([3.0, 0.0]).double(),
         "mix.r2": torch.tensor([2.0, 0.3]).double(),
         "mix.sink": torch.tensor([-2.0, 9.0]).double()}
    mx = {"scale": 1.0, "softcap": 5.0}
    want = _oracle_attn(T, H, G, d, dv, w, q, k, v, mx)
    got = _attn_case(device, T, H, G, d, dv, w, q, k, v, mx)
    torch.testing.assert_close(got.double(), want, atol=2e-4, rtol=2e-4)
    for drop in ("softcap", "sink", "dist"):          # each one is visible
        w2, mx2 = dict(w), dict(mx)
        if drop == "softcap":
            mx2["softcap"] = None
        elif drop == "sink":
            w2["mix.sink"] = torch.tensor([-60.0, -60.0]).double()
        else:
            w2["mix.r1"] = torch.zeros(2).double()
        other = _oracle_attn(T, H, G, d, dv, w2, q, k, v, mx2)
        assert float((other - want).abs().max()) > 0.05


# ---------- whole model ----------

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_logits_and_first_tokens(device, dtype):
    cfg = make_cfg(BASE)
    sd = make_weights(cfg, 1)
    ex = executor(cfg, sd, device, dtype)
    for n in (1, 2, 3, 65):
        toks = tokens(n, cfg["vocab"], n)
        want = O.forward(toks, cfg, sd)
        got = ex.prefill_slots([1], [toks], want=[list(range(n))])[0]
        close(got, want, dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_residual_after_every_layer(device):
    cfg = make_cfg(BASE)
    sd = make_weights(cfg, 2)
    ex = executor(cfg, sd, device)
    toks = tokens(19, cfg["vocab"], 3)
    _, trail = O.forward(toks, cfg, sd, return_layers=True)
    h = ex.model.embed_tokens(toks.view(1, -1).to(ex.device)).clone()
    p0 = torch.zeros(1, dtype=torch.int32, device=ex.device)
    for lid in range(len(BASE)):
        ex.model.prefill_window(h, [lid], ex.kvs[0], p0)
        close(h[0], trail[lid])


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_vs_token_by_token_and_long_decode(device):
    """Prompt of 5, then 200 tokens decoded one by one (crossing the 64-key
    chunk edges of the decode kernel at 63/64/65, 127/128/129, 191/192/193)
    equal the oracle's logits over the whole sequence."""
    cfg = make_cfg(BASE[:2])
    sd = make_weights(cfg, 4)
    ex = executor(cfg, sd, device, slots=3)
    toks = tokens(205, cfg["vocab"], 5)
    want = O.forward(toks, cfg, sd)
    got = ex.prefill_slots([2], [toks[:5]], want=[[4]])[0]
    close(got, want[4:5])
    for i in range(5, 205):
        lg = decode_steps(ex, {2: toks[i]})
        if i in (5, 62, 63, 64, 65, 127, 128, 129, 191, 192, 193, 204):
            close(lg[2:3], want[i:i + 1])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("chunk", [2, 3, 7, 64])
def test_portions(device, chunk):
    cfg = make_cfg(BASE[:3])
    sd = make_weights(cfg, 6)
    ex = executor(cfg, sd, device)
    n = 131
    toks = tokens(n, cfg["vocab"], 7)
    want = O.forward(toks, cfg, sd)
    pick = [0, 1, chunk - 1, chunk, 63, 64, 65, 128, n - 1]
    got = ex.prefill_slots([0], [toks], want=[pick], chunk=chunk)[0]
    close(got, want[pick])
    # a request continued by a further portion, then by single tokens
    ex2 = executor(cfg, sd, device)
    ex2.prefill_slots([3], [toks[:70]], want=[[]])
    got = ex2.prefill_slots([3], [toks[70:129]], want=[[0, 58]],
                            start=[70])[0]
    close(got, want[[70, 128]])
    close(decode_steps(ex2, {3: toks[129]})[3:4], want[129:130])
    close(decode_steps(ex2, {3: toks[130]})[3:4], want[130:131])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_equals_each_alone(device, dtype):
    cfg = make_cfg(BASE)
    sd = make_weights(cfg, 8)
    lens = [1, 67, 30, 128]
    prompts = [tokens(n + 6, cfg["vocab"], 10 + n) for n in lens]
    wants = [O.forward(p, cfg, sd) for p in prompts]
    ex = executor(cfg, sd, device, dtype, slots=5)
    slots = [3, 0, 4, 1]                                # scattered rows
    got = ex.prefill_slots(slots, [p[:n] for p, n in zip(prompts, lens)],
                           want=[list(range(n)) for n in lens])
    for g, w, n in zip(got, wants, lens):
        close(g, w[:n], dtype)
    alive = dict(zip(slots, range(4)))
    for step in range(6):                  # decoded together; short ones
        if step == 3:                      # leave the batch early
            alive.pop(3), alive.pop(4)
        lg = decode_steps(ex, {s: prompts[i][lens[i] + step]
                               for s, i in alive.items()})
        for s, i in alive.items():
            close(lg[s:s + 1], wants[i][lens[i] + step].view(1, -1), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_slot_freed_and_used_again(device):
    cfg = make_cfg(BASE[:2])
    sd = make_weights(cfg, 9)
    ex = executor(cfg, sd, device, slots=2)
    a, b = tokens(90, cfg["vocab"], 1), tokens(40, cfg["vocab"], 2)
    ex.prefill_slots([1], [a], want=[[]])
    for t in tokens(5, cfg["vocab"], 3):
        decode_steps(ex, {1: t})
    ex.kvs[0].pos[1] = 0                                # request ends
    want = O.forward(b, cfg, sd)
    got = ex.prefill_slots([1], [b[:33]], want=[[0, 32]])[0]
    close(got, want[[0, 32]])
    for i in range(33, 40):
        close(decode_steps(ex, {1: b[i]})[1:2], want[i:i + 1])


@pytest.mark.parametrize("device", DEVICES)
def test_other_sizes(device):
    """Sizes the usual configurations make equal or 1: one head, one kv
    head for many heads, dim == vdim, width == ff, embedding scale 1, no
    feed-forward anywhere, a single layer."""
    for layers, kw in (
            ([(mixer(1, 1, 8, 8, scale=1.0), 32)], dict(width=32, emb=1.0)),
            ([(mixer(20, 1, 4, 6), None)] * 2, dict(width=24, vocab=11)),
            ([(mixer(5, 5, 12, 36, softcap=0.7), 130),
              (mixer(2, 1, 64, 2), 8)], dict(width=66, eps=1e-3))):
        cfg = make_cfg(layers, **kw)
        sd = make_weights(cfg, 11)
        ex = executor(cfg, sd, device, slots=2, smax=96)
        toks = tokens(70, cfg["vocab"], 12)
        want = O.forward(toks, cfg, sd)
        got = ex.prefill_slots([0], [toks[:66]], want=[list(range(66))])[0]
        close(got, want[:66])
        for i in range(66, 70):
            close(decode_steps(ex, {0: toks[i]})[0:1], want[i:i + 1])


@pytest.mark.gpu
def test_decode_graph_replays_match_eager():
    """The captured slot-batch decode graph, replayed over many steps with
    eager prefills in between, reproduces the eager steps."""
    cfg = make_cfg(BASE)
    sd = make_weights(cfg, 13)
    toks = tokens(100, cfg["vocab"], 14)
    outs = []
    for graphs in (False, True):
        ex = executor(cfg, sd, "cuda:0", "bfloat16", slots=3, graphs=graphs)
        ex.prefill_slots([0], [toks[:50]], want=[[]])
        got = []
        for i in range(50, 70):
            got.append(decode_steps(ex, {0: toks[i]})[0])
        ex.prefill_slots([2], [toks[:9]], want=[[]])    # eager work between
        torch.cuda.synchronize()
        for i in range(70, 100):
            got.append(decode_steps(ex, {0: toks[i], 2: toks[i - 61]})[0])
        outs.append(torch.stack(got))
    assert torch.equal(outs[0], outs[1])


# ---------- generation through the runtime's scheduler ----------

def write_checkpoint(path: Path, cfg, sd):
    from safetensors.torch import save_file
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in sd.items()},
              str(path / "model.safetensors"))


def oracle_greedy(prompt, n, cfg, sd):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(seq, cfg, sd)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_slot_scheduler(tmp_path, device,
                                                  monkeypatch):
    """Checkpoint on disk -> ShardRuntime load (metadata buckets, weight
    load, slots) -> three concurrent requests of unequal prompts admitted
    as one ragged batch -> greedy tokens equal the oracle's."""
    from dnet_amd.core.types import ShardLoadModelRequest
    from dnet_amd.shard.runtime import ShardRuntime
    cfg = make_cfg(BASE, vocab=61)
    sd = make_weights(cfg, 15)
    write_checkpoint(tmp_path / "m", cfg, sd)
    emitted: dict = {}

    class Cap:
        def send(self, frame):
            emitted.setdefault(frame["nonce"], []).append(
                (frame["token_id"], frame["finished"]))

        def close(self):
            pass

    rt = ShardRuntime("probe")
    # (no repacked-weights cache keyed by a recycled temporary path)
    monkeypatch.setattr(rt.settings.storage, "repack_on_load", False)
    rt._load(ShardLoadModelRequest(
        model_path=str(tmp_path / "m"), total_layers=4, layers=[0, 1, 2, 3],
        max_batch=3, max_seq=128, dtype="float32"))
    assert (rt.executor.device.type == "cuda") == device.startswith("cuda")
    rt._callback = Cap()
    prompts = {"a": tokens(9, 61, 1), "b": tokens(2, 61, 2),
               "c": tokens(31, 61, 3), "d": tokens(5, 61, 4)}
    n_new = {"a": 7, "b": 12, "c": 4, "d": 6}
    for name in ("a", "b", "c", "d"):       # d waits for a slot to free up
        rt.infer_q.put({"nonce": name, "prompt_len": len(prompts[name]),
                        "tokens": prompts[name].to(torch.int32).numpy()
                        .tobytes(), "max_tokens": n_new[name],
                        "stop_ids": [], "params": {}})
    for _ in range(60):
        rt._slots_tick()
        if all(emitted.get(k) and emitted[k][-1][1] for k in prompts):
            break
    for name, p in prompts.items():
        got = [t for t, _ in emitted[name]]
        assert got == oracle_greedy(p.tolist(), n_new[name], cfg, sd), name
    rt._unload()


@pytest.mark.gpu
def test_trace_replay_cli_gpu(tmp_path):
    """The same replay on the GPU box (HIP kernels, captured decode graph,
    slot batch grown after capture)."""
    test_trace_replay_cli(tmp_path)


def test_trace_replay_cli(tmp_path):
    """bin/trace_run end to end on a tiny checkpoint: a prompt batch of
    unequal requests (more of them than the initial slot count, so the slot
    batch grows), decode steps, a request that sits a step out, requests
    that end early."""
    cfg = make_cfg(BASE[:2], vocab=53)
    sd = make_weights(cfg, 16)
    write_checkpoint(tmp_path / "m", cfg, sd)
    a, b = tokens(12, 53, 1).tolist(), tokens(4, 53, 2).tolist()
    c = tokens(7, 53, 3).tolist()
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [0, 8]},
                                {"id": "b", "tokens": b[:2], "want": []},
                                {"id": "c", "tokens": c[:5], "want": [4]}],
         "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[9:10], "want": [0]},
                                {"id": "b", "tokens": b[2:3], "want": [0]}],
         "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[10:11], "want": []},
                                {"id": "b", "tokens": b[3:4], "want": [0]}],
         "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[11:12], "want": [0]}],
         "end": ["a"]},
        {"step": 4, "entries": [{"id": "c", "tokens": c[5:6], "want": [0]}],
         "end": []},
        {"step": 5, "entries": [{"id": "c", "tokens": c[6:7], "want": [0]}],
         "end": ["c"]},
    ]
    root = Path(__file__).resolve().parents[1]
    r = subprocess.run(
        [sys.executable, str(root / "bin" / "trace_run"), "--model",
         str(tmp_path / "m"), "--dtype", "float32", "--out",
         str(tmp_path / "out"), "--max-tokens", "32", "--max-batch", "2"],
        input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
        capture_output=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [
        f"done {i}" for i in range(6)]
    wa, wb = O.forward(a, cfg, sd), O.forward(b, cfg, sd)
    wc = O.forward(c, cfg, sd)
    import numpy as np

    def rd(i):
        return torch.from_numpy(np.fromfile(tmp_path / "out" / f"{i}.f32",
                                            dtype="<f4").reshape(-1, 53))
    close(rd(0), torch.cat([wa[[0, 8]], wc[4:5]]))
    close(rd(1), torch.stack([wa[9], wb[2]]))
    close(rd(2), wb[3:4])
    close(rd(3), wa[11:12])
    close(rd(4), wc[5:6])
    close(rd(5), wc[6:7])


# ---------- pipeline stages (gloo, two processes) ----------

def _ring_tokens():
    g = torch.Generator().manual_seed(21)
    return torch.randint(0, 97, (1, 2, 9), generator=g)


def _ring_run(rank, world):
    mc = ModelConfig.from_hf(make_cfg(BASE))
    mc.compute_dtype = "float32"
    ex = RingExecutor(mc, rank, world, "cpu", mb_count=1, mb_size=2, smax=64,
                      seed=7, use_graphs=False)
    first = ex.prefill(_ring_tokens())
    gen = ex.decode_rounds(5)
    return None if rank else torch.cat([first.unsqueeze(-1), gen], dim=-1)


def _ring_rank_main(rank, world, port, q):
    import os
    os.environ.update(RANK=str(rank), WORLD_SIZE=str(world),
                      MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port),
                      LOCAL_RANK=str(rank))
    import torch.distributed as dist
    dist.init_process_group("gloo", rank=rank, world_size=world)
    out = _ring_run(rank, world)
    if rank == 0:
        q.put(out)
    dist.destroy_process_group()


@pytest.mark.timeout(360)
def test_two_stage_ring_matches_single():
    """Layers split over two pipeline stages: the fp32 residual rides the
    ring hops and the generated tokens equal the single-stage run."""
    import multiprocessing as mp
    import socket
    single = _ring_run(0, 1)
    s = socket.socket()
    s.bind(("127.0.0.1", 0))
    port = s.getsockname()[1]
    s.close()
    ctx = mp.get_context("spawn")
    q = ctx.Queue()
    procs = [ctx.Process(target=_ring_rank_main, args=(r, 2, port, q))
             for r in range(2)]
    for p in procs:
        p.start()
    out = q.get(timeout=150)
    for p in procs:
        p.join(timeout=60)
        assert p.exitcode == 0
    assert torch.equal(out, single)


def test_streamed_weights_match_resident():
    """Windowed weight residency (layers streamed through two device slots)
    generates the same tokens as the fully resident model."""
    cfg = make_cfg([(mixer(4, 2, 16, 8), 40)] * 4)
    toks = torch.randint(0, 97, (1, 2, 9),
                         generator=torch.Generator().manual_seed(1))
    outs = []
    for residency in (0, 2):
        ex = RingExecutor(ModelConfig.from_hf(cfg), 0, 1, "cpu", mb_size=2,
                          smax=64, residency=residency, use_graphs=False)
        first = ex.prefill(toks)
        outs.append(torch.cat([first.unsqueeze(-1), ex.decode_rounds(4)], -1))
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_awkward_sizes(device, dtype):
    """Widths and head sizes that are not multiples of the kernels' vector
    widths or tile sizes: every scalar / padded code path against the
    oracle, in a prompt batch and in decoding."""
    for width, ff, layers in (
            (100, 77, [(mixer(6, 3, 24, 40), 77), (mixer(2, 1, 10, 6), None)]),
            (90, 36, [(mixer(5, 1, 7, 9, softcap=2.0), 36)] * 2),
            (72, 200, [(mixer(3, 3, 72, 136), 200)])):
        cfg = make_cfg(layers, width=width, vocab=131)
        sd = make_weights(cfg, width)
        ex = executor(cfg, sd, device, dtype, slots=3, smax=160)
        a, b = tokens(80, 131, 1), tokens(23, 131, 2)
        wa, wb = O.forward(a, cfg, sd), O.forward(b, cfg, sd)
        got = ex.prefill_slots([2, 0], [a[:70], b[:20]],
                               want=[[0, 31, 32, 63, 64, 69], [0, 19]])
        close(got[0], wa[[0, 31, 32, 63, 64, 69]], dtype)
        close(got[1], wb[[0, 19]], dtype)
        for i in range(3):
            lg = decode_steps(ex, {2: a[70 + i], 0: b[20 + i]})
            close(lg[2:3], wa[70 + i].view(1, -1), dtype)
            close(lg[0:1], wb[20 + i].view(1, -1), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_int8_weights(device):
    """Grouped int8 weights (the framework's W8A16 linears) stay within
    quantization error of the oracle on the unquantized weights."""
    from dnet_amd.models import QuantConfig
    cfg = make_cfg([(mixer(4, 2, 32, 32), 256)] * 2, width=128, vocab=101)
    sd = make_weights(cfg, 31)
    mc = ModelConfig.from_hf(cfg, quant=QuantConfig(8, 128))
    ex = RingExecutor(mc, 0, 1, device, mb_size=2, smax=96,
                      init_weights=False, use_graphs=False)
    ex.model.load_state_dict(sd)
    assert ex.model.layers[0].qkv.is_quant and ex.model.layers[0].down.is_quant
    toks = tokens(40, 101, 5)
    want = O.forward(toks, cfg, sd)
    got = ex.prefill_slots([0], [toks[:36]], want=[[0, 35]])[0]
    scale = float(want.float().pow(2).mean().sqrt())
    assert float((got.float().cpu() - want[[0, 35]].float()).abs().max()) \
        < 0.2 * scale
    lg = decode_steps(ex, {0: toks[36]})
    assert float((lg[0] - want[36].float()).abs().max()) < 0.2 * scale
