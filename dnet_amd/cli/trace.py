"""dnet-trace: replay a token trace through a loaded model and dump logits.

Usage:
  bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Loads the model the way a shard does (ShardRuntime: config -> model class ->
executor -> weights -> KV slots) and then drives the serving step functions
with GIVEN tokens instead of sampled ones: new requests are prefilled as one
ragged slot batch (RingExecutor.prefill_slots), requests that go on by one
token run the slot-batch decode step (RingExecutor.slot_step_compute — the
hipGraph-captured body on a GPU). Nothing is sampled.

Steps arrive on stdin, one JSON object per line:
  {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}],
   "end": []}
For a step with wanted positions the logits go to OUT/<step>.f32
(little-endian fp32 [wanted, vocab], in entry/want order); every step is
acknowledged with a flushed ``done <step>`` line. Requests named in "end"
give their KV slot back. Exit code 3: the requested dtype is not
implemented for this model family.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def main(argv=None) -> int:
    ap = argparse.ArgumentParser("dnet-trace")
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16",
                    choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, default=4096,
                    help="most tokens live requests hold at any time")
    ap.add_argument("--max-batch", type=int, default=8,
                    help="initial KV slot count (grows on demand)")
    ap.add_argument("--gpu-index", type=int, default=0)
    ap.add_argument("--no-graphs", action="store_true")
    args = ap.parse_args(argv)

    if args.dtype == "float32":
        # true fp32 products: no environment override may switch the vendor
        # GEMM to a reduced-precision matrix mode
        import os
        os.environ.pop("TORCH_ALLOW_TF32_CUBLAS_OVERRIDE", None)
    import numpy as np
    import torch
    if args.dtype == "float32":
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False

    on_gpu = torch.cuda.device_count() > 0      # else: CPU reference ops
    if on_gpu:
        from ..ops.build import build, needs_build
        if needs_build():           # fresh checkout: compile the kernels
            print("building the gfx950 extension ...", file=sys.stderr,
                  flush=True)
            build(verbose=False)

    from ..core.types import ShardLoadModelRequest
    from ..models import ModelConfig, get_ring_model
    from ..shard.runtime import ShardRuntime

    hf = json.loads((Path(args.model) / "config.json").read_text())
    cfg = ModelConfig.from_hf(hf)
    cls = get_ring_model(cfg.model_type)
    if args.dtype == "float32" and not getattr(cls, "supports_float32",
                                               False):
        print(f"{cfg.model_type}: no float32 path", file=sys.stderr)
        return 3
    smax = (max(args.max_tokens, 16) + 63) // 64 * 64 + 64
    rt = ShardRuntime("trace")
    # a replay keeps nothing but compiled code between calls: no repacked
    # per-layer weight cache is written or read
    rt.settings.storage.repack_on_load = False
    if args.no_graphs:
        rt.settings.compute.use_graphs = False
    rt._load(ShardLoadModelRequest(
        model_path=args.model, total_layers=cfg.num_layers,
        layers=list(range(cfg.num_layers)), max_batch=max(2, args.max_batch),
        max_seq=smax, dtype=args.dtype, gpu_index=args.gpu_index))
    ex = rt.executor
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)

    slot_of: dict = {}          # request id -> KV slot
    length: dict = {}           # request id -> tokens held so far

    def take_slot() -> int:
        used = set(slot_of.values())
        for s in range(ex.mb_size):
            if s not in used:
                return s
        n = ex.mb_size
        ex.resize_slots(2 * n)
        for name in ("_park_dev", "_free_dev"):
            m = torch.ones(2 * n, dtype=torch.bool, device=ex.device)
            m[:n] = getattr(rt, name)
            setattr(rt, name, m)
        return n

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = step.get("entries", [])
        rows = []
        decode = bool(entries) and all(
            e["id"] in slot_of and len(e["tokens"]) == 1 for e in entries)
        if decode:
            # every request goes on by one token: the slot-batch decode step
            toks = ex.tokbuf[0].cpu()
            for e in entries:
                toks[slot_of[e["id"]]] = int(e["tokens"][0])
            ex.tokbuf[0].copy_(toks)
            # rows that sit this step out (free slots, live requests without
            # an entry) run as idle rows: their recurrent state is kept
            stepped = {slot_of[e["id"]] for e in entries}
            idle = torch.ones(ex.mb_size, dtype=torch.bool)
            idle[sorted(stepped)] = False
            ex.slot_step_compute(park=idle.to(ex.device))
            logits = ex.logits_buf[0].float()
            for e in entries:
                if e.get("want"):
                    rows.append(logits[slot_of[e["id"]]].view(1, -1))
                length[e["id"]] += 1
            ex.slot_advance(rt._park_dev, rt._free_dev)
            # a live request that sat this step out keeps its position (its
            # row ran on a stale token; that append is overwritten by its
            # real next token)
            for rid, s in slot_of.items():
                if s not in stepped:
                    ex.kvs[0].pos[s] = length[rid]
        elif entries:
            slots, prompts, want, start = [], [], [], []
            for e in entries:
                if e["id"] not in slot_of:
                    slot_of[e["id"]] = take_slot()
                    length[e["id"]] = 0
                slots.append(slot_of[e["id"]])
                prompts.append(torch.tensor(e["tokens"], dtype=torch.int64))
                want.append(list(e.get("want", [])))
                start.append(length[e["id"]])
            got = ex.prefill_slots(slots, prompts, want=want, start=start)
            for e, s, lg in zip(entries, slots, got):
                length[e["id"]] += len(e["tokens"])
                rt._park_dev[s] = False
                rt._free_dev[s] = False
                if lg is not None and lg.shape[0]:
                    rows.append(lg.float())
        for rid in step.get("end", []):
            s = slot_of.pop(rid, None)
            length.pop(rid, None)
            if s is not None:
                rt._park_dev[s] = True
                rt._free_dev[s] = True
                ex.kvs[0].pos[s] = 0
        if rows:
            arr = torch.cat(rows).cpu().numpy().astype("<f4")
            tmp = out_dir / f".{step['step']}.part"
            arr.tofile(tmp)
            tmp.rename(out_dir / f"{step['step']}.f32")
        print(f"done {step['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
