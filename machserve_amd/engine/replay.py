"""Trace replay: feeds given token ids through the model step by step and writes logits.
It samples nothing and has no forward pass, cache or loader of its own: it drives the step
function, cache manager and kernels that generation uses.

Input, one JSON object a line:
``{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}``.
For a step that wants something it writes ``<out>/<step>.f32`` (little-endian float32,
``[wanted, vocab]``, in the order of the entries and of their ``want`` lists), and after
every step it prints ``done <step>``.  With a folder for layers it also writes the residual
stream at the wanted places after the embedding and after every run of a layer, as
``<layers>/<step>_embedding.f32`` and ``<layers>/<step>_layer<NN>.f32`` (``[wanted, width]``):
where two runs disagree, the first file that differs names the layer
(``crates/mach-model/src/batched.rs:3040-3088`` is the reference's dump of the same points).

Role in the reference: the test helper ``fwd_rows`` (``crates/mach-model/tests/batched.rs:612-631``).
"""
from __future__ import annotations

import argparse
import json
import os
import sys


from .loading import load_model
from .step import StepEntry


def _write(arr, folder: str, name: str) -> None:
    tmp = os.path.join(folder, f".{name}.tmp")
    arr.detach().to("cpu").float().numpy().astype("<f4", copy=False).tofile(tmp)
    os.replace(tmp, os.path.join(folder, name))


def replay(lm, lines, out_dir: str, say=print, layers_dir=None) -> None:
    slots = {}
    seen = {}
    if layers_dir is not None:
        lm.model.observer = lambda name, stream: seen.__setitem__(name, stream[seen["rows"]].clone())
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if rid not in slots:
                slots[rid] = lm.cache.admit()
            entries.append(StepEntry(slots[rid], e["tokens"], e.get("want", [])))
        if entries:
            if layers_dir is not None:  # the wanted places as rows of the step
                first, rows = 0, []
                for e in entries:
                    rows += [first + w for w in e.want]
                    first += len(e.tokens)
                seen.clear()
                seen["rows"] = rows
            logits = lm.step(entries)
            if logits is not None:
                _write(logits, out_dir, f"{step}.f32")
                for name, rows_of_layer in seen.items():
                    if name != "rows":
                        _write(rows_of_layer, layers_dir, f"{step}_{name}.f32")
        for rid in rec.get("end", []):
            if rid in slots:
                lm.cache.release(slots.pop(rid))
        say(f"done {step}")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True, help="folder the logits are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each rounded up to the page size")
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--dump-layers", default=None, metavar="DIR",
                    help="also write the residual stream at the wanted places after the embedding and after every layer "
                         "(for finding the layer in which two runs part; steps then run from no captured graph)")
    args = ap.parse_args(argv)
    os.makedirs(args.out, exist_ok=True)
    if args.dump_layers:
        os.makedirs(args.dump_layers, exist_ok=True)
    print(f"[trace_run] loading {args.model} as {args.dtype}", file=sys.stderr, flush=True)
    lm = load_model(args.model, dtype=args.dtype, device=args.device, page_size=args.page_size,
                    max_tokens=args.max_tokens, max_requests=64)
    print("[trace_run] ready", file=sys.stderr, flush=True)

    def say(msg):
        sys.stdout.write(msg + "\n")
        sys.stdout.flush()

    # line by line as they arrive: the sender waits for each step's "done" before it writes the next
    replay(lm, iter(sys.stdin.readline, ""), args.out, say, args.dump_layers)
    return 0
