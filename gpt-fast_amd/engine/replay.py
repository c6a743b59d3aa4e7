"""Trace replay: feed given token ids through the engine step by step and write logits.

Nothing is sampled.  The program reads one JSON object per line,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

runs the step through :meth:`Engine.step` (the step function generation uses), writes
``<out>/<step>.f32`` (float32 little-endian, [wanted, vocab], in the order of the entries
and of ``want``) when something is wanted, releases the sequences named in ``end``, and
prints ``done <step>``.  The reference has no such program; its nearest relatives are the
whole-sequence call of eval.py:134-148 and the multi-token step at an offset of
generate.py:104-108.
"""
import argparse
import json
import os
import sys
from typing import Dict

import torch

from .batch import Entry
from .step import Engine


def replay(engine: Engine, lines, out_dir: str, log=None) -> int:
    os.makedirs(out_dir, exist_ok=True)
    slots: Dict[str, int] = {}
    keys: Dict[str, int] = {}
    steps = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for item in rec.get("entries", []):
            rid = str(item["id"])
            if rid not in slots:
                slots[rid] = engine.start_sequence()
                keys[rid] = len(keys)
            entries.append(Entry(slot=slots[rid], tokens=[int(t) for t in item["tokens"]],
                                 want=[int(i) for i in item.get("want", [])], key=keys[rid]))
        if entries:
            logits = engine.step(entries)
            if logits.shape[0] > 0:
                data = logits.detach().to("cpu", torch.float32).contiguous().numpy()
                path = os.path.join(out_dir, f"{step}.f32")
                with open(path + ".tmp", "wb") as f:
                    data.astype("<f4", copy=False).tofile(f)
                os.replace(path + ".tmp", path)
            else:
                torch.cuda.synchronize()
        for rid in rec.get("end", []):
            rid = str(rid)
            if rid not in slots:
                raise KeyError(f"step {step}: request '{rid}' ends but was never started")
            engine.end_sequence(slots.pop(rid))
        print(f"done {step}", flush=True)
        steps += 1
    return steps


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each rounded up to 64")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    engine = Engine.from_folder(args.model, dtype=args.dtype, device=args.device,
                                max_tokens=args.max_tokens)
    replay(engine, sys.stdin, args.out)
    return 0
