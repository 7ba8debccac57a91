"""Replay a recorded token schedule through the serving engine and write
the logits it produces.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Reads one JSON object per line from standard input:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Each entry feeds a request's next tokens (a request is admitted at its first
entry; it may skip steps); all entries of a step run as ONE engine batch,
prompt portions beside single tokens. ``want`` lists the places among the
entry's tokens whose logits are written, in entry order, to
``<out>/<step>.f32`` as little-endian float32 [wanted, vocab]. ``end`` names
requests whose state slot and KV pages are released after the step. After
every step the line ``done <step>`` is printed.

Nothing is sampled: this is the engine's generation step
(:meth:`ServingEngine.forced_step` — same model forward, paged KV cache,
recurrent-state slots and kernels) driven with given tokens, which makes it
a tool for comparing engines or precisions position by position. The page
pool holds ``--max-tokens`` tokens in 64-token pages and there are four
sequence slots, so long schedules recycle both.
"""

from __future__ import annotations

import argparse
import json
import os
import sys

MAX_LIVE = 4
PAGE = 64


def build_engine(model_dir: str, dtype: str, max_tokens: int, device=None):
    import torch

    from neuronx_distributed_inference_amd.config import EngineConfig
    from neuronx_distributed_inference_amd.registry import (
        get_model_classes,
        model_type_from_config,
    )
    from neuronx_distributed_inference_amd.serving import ServingEngine

    if device is None:
        device = torch.device("cuda", 0) if torch.cuda.is_available() else torch.device("cpu")
    if dtype == "float32":
        # true 32-bit products: no reduced-precision matrix modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    model_type = model_type_from_config(model_dir)
    config_cls, model_cls = get_model_classes(model_type)
    pages = (max_tokens + PAGE - 1) // PAGE
    ec = EngineConfig(
        batch_size=MAX_LIVE, max_batch_size=MAX_LIVE, kv_cache_batch_size=MAX_LIVE,
        seq_len=pages * PAGE, max_length=pages * PAGE, torch_dtype=dtype,
        tp_degree=1, is_block_kv_layout=True, pa_block_size=PAGE,
        pa_num_blocks=pages, enable_hip_graphs=False, output_logits=True,
    )
    config = config_cls.from_hf_config(model_dir, neuron_config=ec)
    model = model_cls.from_pretrained(model_dir, config).to(device).eval()
    engine = ServingEngine(model, max_slots=MAX_LIVE, capture_decode=False, async_depth=1)
    return engine


def replay(engine, lines, out_dir: str, emit=print):
    import numpy as np
    import torch

    live = {}
    with torch.no_grad():
        for line in lines:
            line = line.strip()
            if not line:
                continue
            msg = json.loads(line)
            parts, wants = [], []
            for e in msg.get("entries", []):
                req = live.get(e["id"])
                if req is None:
                    req = live[e["id"]] = engine.admit()
                if not e.get("tokens"):
                    continue                  # admitted, nothing to feed yet
                parts.append((req, torch.tensor(e["tokens"], dtype=torch.long)))
                wants.append(e.get("want", []))
            if parts:
                logits = engine.forced_step(parts)
                rows = [logits[i, w] for i, ws in enumerate(wants) for w in ws]
                if rows:
                    arr = torch.stack(rows).float().cpu().numpy().astype("<f4")
                    tmp = os.path.join(out_dir, ".%d.part" % msg["step"])
                    arr.tofile(tmp)
                    os.replace(tmp, os.path.join(out_dir, "%d.f32" % msg["step"]))
            for rid in msg.get("end", []):
                req = live.pop(rid, None)
                if req is not None:
                    engine.release(req)
            emit("done %d" % msg["step"])


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--cpu", action="store_true", help="run the reference ops on the CPU")
    args = ap.parse_args(argv)
    # a replay sees arbitrary batch shapes once each: per-shape timed GEMM
    # autotuning would cost more than it saves
    os.environ.setdefault("NXDI_DISABLE_HIPBLASLT", "1")
    import torch

    os.makedirs(args.out, exist_ok=True)
    device = torch.device("cpu") if args.cpu else None
    engine = build_engine(args.model, args.dtype, args.max_tokens, device)

    def emit(s):
        sys.stdout.write(s + "\n")
        sys.stdout.flush()

    replay(engine, sys.stdin, args.out, emit)
    return 0


if __name__ == "__main__":
    sys.exit(main())
