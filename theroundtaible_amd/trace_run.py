"""Replay a token trace through the engine, step by step, and write the logits that are asked for.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

``DIR`` holds ``config.json`` (its ``architecture`` names the model class) and
``model.safetensors``. Steps arrive on standard input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry gives a request's NEXT tokens (a whole prompt, a portion of one, or one decoded
token) and the places among them whose logits are wanted; all entries of a step run as one
batch through :meth:`Engine.step`. Requests named in ``end`` give their cache blocks and state
slot back after the step. For a step with wanted rows the logits are written to
``<out>/<step>.f32`` (little-endian float32, [wanted, vocab], entry order); after every step the
line ``done <step>`` is printed. Nothing is sampled.

The cache pool holds ``--max-tokens`` tokens (each live request rounded up to whole pages) and
``--max-live`` state slots, so pages and slots are reused as requests end.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="checkpoint directory (config.json + model.safetensors)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="directory for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens live requests hold at any time")
    ap.add_argument("--max-live", type=int, default=4, help="requests live at any time (state slots)")
    ap.add_argument("--device", default=None, help="default: cuda:0 (cpu runs the PyTorch statements of the ops)")
    ap.add_argument("--block-size", type=int, default=64)
    a = ap.parse_args(argv)

    import torch
    device = a.device or ("cuda:0" if torch.cuda.is_available() else None)
    if device is None:
        print("trace_run: no GPU visible (pass --device cpu to run the reference ops)", file=sys.stderr)
        return 2
    from .engine import Engine, EngineConfig
    from .models.config import get_config
    from .utils.local_detect import resolve_model
    # the checkpoint's config.json names the model class, as for every engine built on a directory
    model, overrides = resolve_model(a.model, a.model)
    if device.startswith("cuda"):      # a fresh checkout compiles the model family's kernels here, once
        arch = get_config(model, **overrides).arch
        if arch == "mupulorn":
            from .ops import latent
            latent.ensure_built()
        elif arch in ("goganex", "retuvik", "ledinex"):
            from .ops import hybrid
            hybrid.ensure_built()
    bs = a.block_size
    live = max(1, a.max_live)
    engine = Engine(EngineConfig(model=model, model_overrides=overrides, weights=a.model, dtype=a.dtype, device=device, block_size=bs,
                                 num_blocks=(a.max_tokens + bs - 1) // bs, use_graphs=False, state_slots=live,
                                 max_batch=live))
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
                   for e in st["entries"]]
        logits = engine.step(entries, end=st.get("end", []))
        if logits.shape[0]:
            tmp = os.path.join(a.out, f".{st['step']}.part")
            with open(tmp, "wb") as f:
                f.write(logits.detach().to("cpu").contiguous().numpy().astype("<f4").tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        sys.stdout.write(f"done {st['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
