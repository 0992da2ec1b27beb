"""Trace replay: feed given token ids through a model step by step and write logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Reads one JSON object per line from standard input,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

runs each step's entries as one batch through LLMEngine.replay_step (the engine's scheduler
and block manager, the model runner's mixed and hipGraph decode paths, the model's kernels),
writes DIR/<step>.f32 -- little-endian fp32 [wanted, vocab] -- when something is wanted, and
prints `done <step>` after every step.  The KV pool holds --max-tokens tokens and there are
--max-seqs sequence slots: blocks and slots of ended requests are used again.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np


def build_engine(model: str, dtype: str, max_tokens: int, max_seqs: int = 4,
                 block_size: int = 32, device: str = "auto", enforce_eager: bool = False,
                 log=None):
    from .config import EngineConfig
    from .llm_engine import LLMEngine

    blocks = -(-max_tokens // block_size)
    ecfg = EngineConfig(
        model=model, load_format="safetensors", weights_path=model, dtype=dtype,
        max_model_len=blocks * block_size, max_num_seqs=max_seqs,
        max_num_batched_tokens=blocks * block_size, block_size=block_size,
        num_gpu_blocks=blocks, enable_prefix_caching=False, enforce_eager=enforce_eager,
        device=device, logits_only=True, gc_freeze=False)
    return LLMEngine(ecfg, log=log or (lambda *a: print(*a, file=sys.stderr, flush=True)))


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json + model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="tokens the KV pool holds (rounded up to whole blocks)")
    ap.add_argument("--max-seqs", type=int, default=4, help="sequence slots")
    ap.add_argument("--block-size", type=int, default=32)
    ap.add_argument("--device", default=os.environ.get("AKAP_DEVICE", "auto"))
    ap.add_argument("--enforce-eager", action="store_true", help="no hipGraph decode")
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    eng = build_engine(a.model, a.dtype, a.max_tokens, a.max_seqs, a.block_size, a.device,
                       a.enforce_eager)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want") or []) for e in st["entries"]]
        logits = eng.replay_step(entries, st.get("end") or [])
        if logits.shape[0]:
            tmp = os.path.join(a.out, f".{st['step']}.part")
            np.ascontiguousarray(logits, dtype="<f4").tofile(tmp)
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        print(f"done {st['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
