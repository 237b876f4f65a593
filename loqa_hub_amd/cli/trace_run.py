"""Replay a token trace through the LLM engine and write logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

``DIR`` holds config.json and model.safetensors; the model family is chosen by
config.json (``models/registry.py``). Steps arrive on standard input, one JSON
object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step are one engine step (``LLMEngine.step_logits``): prompt
portions beside single tokens, on top of what the paged cache and the state
slots hold from earlier steps. The logits at the wanted places go to
``<out>/<step>.f32`` (little-endian f32 [wanted, vocab], entries in order);
every step answers ``done <step>``. The cache pool holds ``--max-tokens``
tokens and four sequences at a time; ``end`` gives a sequence's pages and slot
back. Nothing is sampled.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

MAX_LIVE = 4


def build_engine(model_dir: str, dtype: str, max_tokens: int, device=None, block_size: int = 16):
    import torch

    from ..engine.llm_engine import LLMEngine
    from ..models.registry import family_of, lm_config_of_checkpoint, load_lm_weights
    dt = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    cfg = lm_config_of_checkpoint(model_dir, os.path.basename(os.path.normpath(model_dir)))
    if dt == torch.float32 and not family_of(cfg).hybrid:
        raise SystemExit(3)          # that family is served in bfloat16 only
    if device is None:
        device = "cuda:0" if torch.cuda.is_available() else "cpu"
    if dt == torch.float32:
        # true 32-bit matrix products
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    cap = -(-max_tokens // block_size) * block_size
    weights = load_lm_weights(cfg, model_dir, device, dtype=dt, max_positions=cap)
    return LLMEngine(cfg, device, weights=weights, max_seqs=MAX_LIVE, max_seq_len=cap,
                     block_size=block_size, num_blocks=cap // block_size, use_graphs=False,
                     dtype=dt)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--device", default=None)
    a = ap.parse_args(argv)
    import numpy as np
    import torch
    os.makedirs(a.out, exist_ok=True)
    eng = build_engine(a.model, a.dtype, a.max_tokens, a.device)
    live: dict[str, object] = {}
    with torch.inference_mode():
        for line in sys.stdin:
            line = line.strip()
            if not line:
                continue
            st = json.loads(line)
            entries = st.get("entries", [])
            seqs, feeds, want = [], [], []
            for e in entries:
                if e["id"] not in live:
                    live[e["id"]] = eng.open_sequence()
                if not e["tokens"]:
                    continue
                seqs.append(live[e["id"]])
                feeds.append([int(t) for t in e["tokens"]])
                want.append([int(w) for w in e.get("want", [])])
            if seqs:
                logits = eng.step_logits(seqs, feeds, want)
                if logits.shape[0]:
                    arr = logits.detach().to("cpu", torch.float32).numpy().astype("<f4")
                    tmp = os.path.join(a.out, f".{st['step']}.part")
                    arr.tofile(tmp)
                    os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
                elif eng.is_gpu:
                    torch.cuda.synchronize(eng.device)
            for i in st.get("end", []):
                r = live.pop(i, None)
                if r is not None:
                    eng.close_sequence(r)
            sys.stdout.write(f"done {st['step']}\n")
            sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
