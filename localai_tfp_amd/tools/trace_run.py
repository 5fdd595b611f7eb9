"""Replay a trace of engine steps and write logits: the tool behind `bin/trace_run` and `local-ai util trace-run`.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N [--max-seqs 4] [--device cuda]

Standard input carries one JSON object per line,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}
Each line is ONE engine step (LLMEngine.replay_step): every entry brings a request's next tokens, all entries run as
one batch from the cache and state earlier steps left, and `want` lists the positions among an entry's tokens whose
logits are written to OUT/<step>.f32 (little-endian fp32 [wanted, vocab], in entry order; no file when nothing is
wanted). `end` names the requests that are finished after the step. After each step it prints `done <step>`.

The engine's cache pool holds --max-tokens tokens (each live request rounded up to whole blocks) and --max-seqs
state slots; nothing is sampled. The model class follows config.json, as for serving (models/loader.py).
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-seqs", type=int, default=4)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--device", default="cuda", help="cuda (default), or cpu for the fp32 plumbing path without kernels")
    a = ap.parse_args(argv)

    import numpy as np
    import torch
    from ..engine.engine import EngineConfig, LLMEngine
    from ..models.loader import load_llm

    dev = a.device
    if dev.startswith("cuda"):  # the model's kernel library is built at its first launch if the tree has none
        if not torch.cuda.is_available():  # never a silent CPU run: the kernels are what a replay is about
            print("trace_run: no GPU is visible (pass --device cpu for the plumbing path)", file=sys.stderr)
            return 2
        torch.backends.cuda.matmul.allow_tf32 = False
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[a.dtype]
    model, tok, _cfg, _ = load_llm(a.model, torch.device(dev), overrides={"dtype": dtype})
    if not hasattr(model, "cache_kind"):
        print("trace_run: this model family has no replayable engine path", file=sys.stderr)
        return 3
    bs = a.block_size
    cfg = EngineConfig(max_num_seqs=a.max_seqs, max_batched_tokens=max(a.max_tokens, a.max_seqs),
                       max_model_len=a.max_tokens, block_size=bs, num_blocks=-(-a.max_tokens // bs) + 1,
                       enable_prefix_cache=False, use_graphs=False, overlap=False, native_scheduler=False,
                       logits_rows=a.max_tokens, gemm_autotune=False)
    eng = LLMEngine(model, tok, cfg)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = eng.replay_step([(e["id"], e["tokens"], e.get("want") or []) for e in st.get("entries", [])],
                                 st.get("end") or [])
        if logits is not None:
            tmp = os.path.join(a.out, ".%s.part" % st["step"])
            np.ascontiguousarray(logits.numpy(), dtype="<f4").tofile(tmp)
            os.replace(tmp, os.path.join(a.out, "%s.f32" % st["step"]))
        print("done %s" % st["step"], flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
