"""Replay a recorded schedule through the engine and dump logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}],
     "end": ["a"]}

Every entry carries a request's next tokens; all entries of a step run as one
engine batch (`LLMEngine.replay_step`: the scheduler admits the requests and
grows their pages and state slots, the model runs the batch with the same
kernels and decode graphs generation uses; nothing is sampled). For a step
with wanted positions the fp32 logits [wanted, vocab] go to OUT/<step>.f32 in
entry order; after every step a line `done <step>` is printed. Requests named
in `end` give their pages and state slot back.
"""

from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True,
                    help="directory with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"],
                    default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="tokens the cache pool must hold at any one time")
    ap.add_argument("--max-seqs", type=int, default=4,
                    help="sequences (and state slots) live at any one time")
    ap.add_argument("--device", default=None)
    ap.add_argument("--eager", action="store_true",
                    help="do not capture decode steps into hipGraphs")
    args = ap.parse_args(argv)

    import torch

    device = args.device or ("cuda" if torch.cuda.is_available() else "cpu")
    if device.startswith("cuda"):
        from ..build import ensure_built

        ensure_built(["_C_mix"])
    # true fp32 GEMMs when serving in fp32
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")

    from ..models.registry import spec_from_dir
    from .config import KV_BLOCK_SIZE, EngineConfig
    from .engine import LLMEngine

    spec = spec_from_dir(args.model)
    bs = KV_BLOCK_SIZE
    # each live request may round its length up to a whole page
    blocks = (args.max_tokens + bs - 1) // bs + 1   # + the scratch page
    cfg = EngineConfig(
        spec=spec, device=device,
        dtype=torch.bfloat16 if args.dtype == "bfloat16" else torch.float32,
        max_model_len=max(bs, args.max_tokens), max_num_seqs=args.max_seqs,
        num_kv_blocks=blocks, max_tokens_per_step=max(1, args.max_tokens),
        enforce_eager=args.eager)
    eng = LLMEngine(cfg)
    os.makedirs(args.out, exist_ok=True)
    sys.stdout.write(f"engine {spec.arch} on {device} in {args.dtype}, "
                     f"{blocks} pages of {bs}\n")
    sys.stdout.flush()

    live = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = []
        for e in step["entries"]:
            req = live.get(e["id"])
            if req is None:
                req = live[e["id"]] = eng.new_replay_request()
            entries.append((req, e["tokens"], e.get("want", [])))
        logits = eng.replay_step(entries)
        if logits is not None:
            data = logits.detach().to("cpu", torch.float32).contiguous().numpy()
            tmp = os.path.join(args.out, f".{step['step']}.part")
            with open(tmp, "wb") as f:
                f.write(data.astype("<f4").tobytes())
            os.replace(tmp, os.path.join(args.out, f"{step['step']}.f32"))
        elif device.startswith("cuda"):
            torch.cuda.synchronize()
        for name in step.get("end", []):
            req = live.pop(name, None)
            if req is not None:
                eng.finish_replay_request(req)
        sys.stdout.write(f"done {step['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
