"""Replay a token trace through the continuous-batching engine and write logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object per line:
``{"step": n, "entries": [{"id": ..., "tokens": [...], "want": [...]}], "end": [...]}``.
All entries of a step run as ONE ragged engine step (prompt portions next to
single decode tokens) on the caches that earlier steps left; ``want`` lists the
places among an entry's tokens whose logits are written, as little-endian
float32 ``[wanted, vocab]``, to ``<out>/<step>.f32``. Requests named in ``end``
give back their pages and state slot after the step. ``done <step>`` is printed
after every step. Nothing is sampled. The KV pool is sized for ``--max-tokens``
live tokens (each request rounded up to whole pages) and ``--slots`` sequences,
so pages and slots are reused as requests come and go.
"""

import argparse
import json
import os
import sys

import torch


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--slots", type=int, default=4, help="sequences that can be live at once")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--device", default=None)
    a = ap.parse_args(argv)

    from ..models import load_pretrained
    from .config import InferenceConfig
    from .paged_engine import ContinuousBatchEngine

    dtype = torch.float32 if a.dtype == "float32" else torch.bfloat16
    device = a.device or ("cuda" if torch.cuda.is_available() else "cpu")
    if dtype == torch.float32:
        # true 32-bit products: no reduced-precision matrix mode
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    model = load_pretrained(a.model, dtype=dtype, device=device)
    if not getattr(model, "serves_ragged", False):
        print(f"{type(model).__name__} has no ragged serving step to replay a trace through", file=sys.stderr)
        return 4
    page = a.page_size
    # a request's share is rounded up to 64 tokens by the caller; whole pages of ours fit into that
    pages = (a.max_tokens + page - 1) // page
    engine = ContinuousBatchEngine(model, InferenceConfig(max_batch_size=a.slots, dtype=dtype),
                                   num_blocks=pages, block_size=page)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        items = [(e["id"], e["tokens"], e.get("want") or []) for e in step["entries"] if e["tokens"]]
        if items:
            logits = engine.run_ragged(items)
            if logits.shape[0]:
                data = logits.to(torch.float32).cpu().contiguous().numpy().astype("<f4")
                tmp = os.path.join(a.out, ".%s.part" % step["step"])
                with open(tmp, "wb") as f:
                    f.write(data.tobytes())
                os.replace(tmp, os.path.join(a.out, "%s.f32" % step["step"]))
        for seq_id in step.get("end") or []:
            engine.close_sequence(seq_id)
        sys.stdout.write("done %s\n" % step["step"])
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
