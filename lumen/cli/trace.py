"""``trace_run``: replay a token trace through the serving engine and write the logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Reads one JSON object per line on standard input,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
runs the step's entries as one engine batch (``lumen.serve.trace.TraceReplay``), writes the
wanted logits to ``<out>/<step>.f32`` (little-endian fp32 [wanted, vocab]; no file when nothing
is wanted) and answers ``done <step>`` on standard output.  The cache pool holds ``--max-tokens``
tokens (in blocks of ``--block-size``) and ``--max-seqs`` requests may be live at a time.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def build_parser():
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="directory with config.json + model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "float16"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-seqs", type=int, default=4)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--no-graphs", action="store_true", help="run decode steps eagerly")
    ap.add_argument("--device", default=None)
    return ap


def main(argv=None) -> int:
    a = build_parser().parse_args(argv)
    import numpy as np
    import torch

    from ..serve.engine import EngineConfig, LLMEngine
    from ..serve.trace import TraceReplay

    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    os.makedirs(a.out, exist_ok=True)
    bs = a.block_size
    blocks = (a.max_tokens + bs - 1) // bs
    eng = LLMEngine(EngineConfig(
        model=a.model, dtype={"bfloat16": "bf16", "float32": "fp32", "float16": "fp16"}[a.dtype],
        max_model_len=max(bs, a.max_tokens), block_size=bs, num_blocks=blocks,
        max_num_seqs=a.max_seqs, max_num_batched_tokens=max(bs, a.max_tokens),
        use_graphs=not a.no_graphs, async_scheduling=False, device=a.device, init="pretrained"))
    replay = TraceReplay(eng)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = replay.step(st.get("entries", []), st.get("end", []))
        if logits.shape[0]:
            tmp = os.path.join(a.out, f".{st['step']}.part")
            np.ascontiguousarray(logits.numpy().astype("<f4")).tofile(tmp)
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        sys.stdout.write(f"done {st['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
