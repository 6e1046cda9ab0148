"""Generate from a checkpoint folder on the command line.

    bin/ds_generate --model-dir DIR --tokens 5,17,3 [--tokens 9,9] \\
        --max-new-tokens 32 [--sample --temperature 0.8 --top-k 50 --top-p 0.95]

``config.json`` names the architecture (models/registry.py). Every ``--tokens``
is one prompt (token ids, comma separated); the prompts are served together by
``init_inference(...).generate``. Prints one JSON line per prompt.
"""

import argparse
import json
import sys

import torch


def main(argv=None):
    ap = argparse.ArgumentParser(prog="ds_generate")
    ap.add_argument("--model-dir", required=True)
    ap.add_argument("--tokens", action="append", required=True,
                    help="one prompt: comma-separated token ids (repeatable; "
                         "prompts of one call have equal length)")
    ap.add_argument("--max-new-tokens", type=int, default=32)
    ap.add_argument("--dtype", default="bfloat16",
                    choices=["bfloat16", "float32"])
    ap.add_argument("--sample", action="store_true")
    ap.add_argument("--temperature", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--eos", type=int, default=None)
    a = ap.parse_args(argv)

    import deepspeed_amd
    from ..models.registry import load_pretrained
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[a.dtype]
    device = "cuda" if torch.cuda.is_available() else "cpu"
    model = load_pretrained(a.model_dir, dtype=dtype, device=device)
    engine = deepspeed_amd.init_inference(model, dtype=dtype)
    prompts = [[int(x) for x in t.split(",")] for t in a.tokens]
    if len({len(p) for p in prompts}) != 1:
        ap.error("prompts of one call must have equal length")
    ids = torch.tensor(prompts, dtype=torch.long)
    out = engine.generate(ids, max_new_tokens=a.max_new_tokens,
                          do_sample=a.sample, temperature=a.temperature,
                          top_k=a.top_k, top_p=a.top_p, eos_token_id=a.eos)
    for p, row in zip(prompts, out.tolist()):
        print(json.dumps({"prompt": p, "generated": row[len(p):]}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
