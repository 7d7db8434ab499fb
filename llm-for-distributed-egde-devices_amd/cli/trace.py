"""Trace replay: feed given token ids through a model step by step and write the logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object per line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step run as one ragged batch through ``engine.ragged.RaggedEngine`` (the step
function the scheduler and ``generate`` use): prompt portions beside single decode tokens.  For a
step that wants logits, ``<out>/<step>.f32`` receives them as little-endian fp32 [wanted, vocab]
in entry order; every step is acknowledged with a flushed ``done <step>`` line.  ``end`` lists the
requests whose slot and pages are given back after the step.  Nothing is sampled.

``--max-tokens`` sizes the page pool (tokens alive at one time, each request rounded up to a
page); ``--slots`` the number of live requests.  Exit code 3: the model cannot run in the
requested dtype.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import torch


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--slots", type=int, default=4)
    ap.add_argument("--device", default=None, help="default: cuda:0 when a GPU is present")
    a = ap.parse_args(argv)

    from .. import ops
    from ..engine.ragged import RaggedEngine
    from ..models.registry import load_model

    # this program runs ragged-step models only: their kernels are a library of their own, built on
    # first use; the projections take the vendor GEMM when the main kernel library was never built
    ops.require_main_ext(False)

    dev = torch.device(a.device) if a.device else torch.device("cuda:0" if torch.cuda.is_available() else "cpu")
    torch.backends.cuda.matmul.allow_tf32 = False            # float32 means fp32 products
    model, _, _ = load_model(a.model, precision={"bfloat16": "bf16", "float32": "fp32"}[a.dtype], device=dev)
    if not getattr(model, "ragged", False):
        sys.stderr.write("trace replay needs a ragged-step (layer-spec) model\n")
        return 3
    if {"bfloat16": torch.bfloat16, "float32": torch.float32}[a.dtype] != model.dtype:
        return 3
    eng = RaggedEngine(model, a.max_tokens, slots=a.slots)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want") or []) for e in st["entries"]]
        logits = eng.step(entries)
        if logits.shape[0]:
            data = logits.to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
            tmp = os.path.join(a.out, f".{st['step']}.part")
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        elif dev.type == "cuda":
            torch.cuda.synchronize()
        for rid in st.get("end") or []:
            if rid in eng.live:
                eng.close(rid)
        sys.stdout.write(f"done {st['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
