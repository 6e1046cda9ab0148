"""Replay a recorded serving schedule through the continuous batcher.

Input (stdin): one JSON object per line,
``{"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}``. All
entries of a step are one ragged batch fed to ``ContinuousBatcher.feed``; a
request is admitted at its first entry and its slot and blocks are given back
when it is listed in ``end``. For a step that wants logits, ``<out>/<n>.f32``
receives them as little-endian fp32 ``[wanted, vocab]``; every step is
acknowledged with ``done <n>`` on stdout. Nothing is sampled.
"""

import argparse
import json
import os
import sys

import torch


def main(argv=None):
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="tokens live at once, per request rounded up to the block size")
    ap.add_argument("--slots", type=int, default=4)
    ap.add_argument("--device", default=None)
    a = ap.parse_args(argv)

    from ..models.registry import load_pretrained
    from .ragged import ContinuousBatcher

    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[a.dtype]
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    device = a.device or ("cuda" if torch.cuda.is_available() else "cpu")
    model = load_pretrained(a.model, dtype=dtype, device=device)
    if not hasattr(model, "build_cache"):
        sys.stderr.write("this architecture has no ragged step\n")
        return 3
    batcher = ContinuousBatcher(model, max_slots=a.slots, dtype=dtype,
                                device=torch.device(device),
                                max_tokens=a.max_tokens)
    os.makedirs(a.out, exist_ok=True)
    live = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries, rows, at = [], [], 0
        for e in step["entries"]:
            if e["id"] not in live:
                live[e["id"]] = batcher.open(e["id"])
            if not e["tokens"]:
                continue                 # admitted, nothing to run yet
            entries.append((live[e["id"]], e["tokens"]))
            rows += [at + w for w in e.get("want", [])]
            at += len(e["tokens"])
        if entries:
            logits = batcher.feed(entries, rows=rows if rows else [0])
            if rows:
                buf = logits.float().cpu().contiguous().numpy().astype("<f4")
                tmp = os.path.join(a.out, ".%d.part" % step["step"])
                with open(tmp, "wb") as f:
                    f.write(buf.tobytes())
                os.replace(tmp, os.path.join(a.out, "%d.f32" % step["step"]))
            elif logits.is_cuda:
                torch.cuda.synchronize()
        for i in step.get("end", []):
            if i in live:
                batcher.close(live.pop(i))
        sys.stdout.write("done %d\n" % step["step"])
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
