"""Replay a token trace through the rollout engine and write logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:
``{"step": 0, "entries": [{"id": "a", "tokens": [5, 17], "want": [1]}],
"end": []}``.  All entries of a step run as one batch through
``Engine.step_forced`` (the engine's model, cache pool, state slots and
kernels; nothing is sampled).  For a step that wants logits the file
``<out>/<step>.f32`` holds them as little-endian fp32 [wanted, vocab]; every
step is acknowledged with a ``done <step>`` line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run")
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16",
                    choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--slots", type=int, default=4,
                    help="requests live at any time (state slots)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--device", default=None)
    a = ap.parse_args(argv)

    import torch
    from polyrl_amd.rollout.loader import engine_from_dir
    device = a.device or ("cuda" if torch.cuda.is_available() else "cpu")
    dtype = getattr(torch, a.dtype)
    if dtype == torch.float32:
        # true fp32 products: no reduced-precision matrix modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    # every live request may round its count up to a multiple of 64
    engine = engine_from_dir(a.model, device=device, dtype=dtype,
                             page_size=a.page_size,
                             kv_token_capacity=a.max_tokens,
                             max_running_requests=a.slots,
                             max_num_batched_tokens=1 << 30)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", []))
                   for e in st["entries"]]
        logits = engine.step_forced(entries, st.get("end", []))
        if logits is not None:
            arr = logits.float().cpu().contiguous().numpy().astype("<f4")
            tmp = os.path.join(a.out, ".%s.part" % st["step"])
            with open(tmp, "wb") as f:
                f.write(arr.tobytes())
            os.replace(tmp, os.path.join(a.out, "%s.f32" % st["step"]))
        sys.stdout.write("done %s\n" % st["step"])
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
