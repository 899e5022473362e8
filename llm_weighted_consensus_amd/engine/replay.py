"""Replay a token trace through the engine, step by step, and write the logits asked for.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input: one JSON object a line,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
Each step's entries are one batch of :meth:`LLMEngine.step_tokens` (the engine's block manager, paged cache and
the model's mixed forward: prompt portions beside single next tokens); nothing is sampled.  For a step that wants
logits, ``<out>/<step>.f32`` holds them as little-endian fp32 [wanted, vocab], entries and wanted places in the
given order.  After every step one line ``done <step>`` goes to standard output.  The cache pool is sized for
``--max-tokens`` tokens held at once (each sequence rounded up to whole pages), so pages are used again as
sequences end.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the live sequences hold at most")
    ap.add_argument("--max-seqs", type=int, default=4, help="sequences alive at once")
    ap.add_argument("--block-size", type=int, default=16)
    a = ap.parse_args(argv)

    import numpy as np
    import torch

    from .. import _build
    from ..models.registry import DTYPES, load_model

    if not _build.RUNTIME_SO.exists():  # a fresh checkout: the host runtime (g++) first; kernels build on first use
        _build.build_runtime()
    from .engine import LLMEngine
    from .tokenizer import load_tokenizer

    if not torch.cuda.is_available():
        print("trace_run: no GPU visible", file=sys.stderr)
        return 2
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    bs = a.block_size
    pad = 64 if 64 % bs == 0 else bs
    max_len = -(-a.max_tokens // pad) * pad
    model = load_model(a.model, device=dev, dtype=DTYPES[a.dtype], max_position=max_len)
    if not hasattr(model, "forward_mixed"):
        print("trace_run: this model has no mixed forward", file=sys.stderr)
        return 2
    eng = LLMEngine(model, load_tokenizer({}, model.cfg.vocab_size), block_size=bs, num_blocks=max_len // bs,
                    max_batch=a.max_seqs, max_model_len=max_len, use_graphs=False, prefix_sharing=False, tune_gc=False)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", [])) for e in st["entries"]]
        logits = eng.step_tokens(entries, st.get("end", ()))
        if logits is not None:
            arr = logits.detach().to(torch.float32).cpu().numpy().astype("<f4", copy=False)
            tmp = os.path.join(a.out, f".{st['step']}.part")
            with open(tmp, "wb") as f:
                f.write(np.ascontiguousarray(arr).tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        print(f"done {st['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
