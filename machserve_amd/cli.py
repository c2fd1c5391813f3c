"""Command line: generation from token ids, ``doctor`` and ``--version``.

Options carry the reference's names and meanings where it has them.  The reference's
binary is configured through the environment (``crates/mach-server/src/main.rs:6-37,
399-453``); each of those variables is the default of the option of the same name here:
MACH_MODEL (--model), MACH_DTYPE (--dtype), MACH_CAPACITY (--capacity, requests running at
once, 64), MACH_PREFILL_ROWS (--prefill-rows, tokens per step, 512), MACH_TPP (--tpp, tokens
per page, 64), MACH_MAX_SEQ (--max-seq, longest request).  Sampling options are those of
its ``SamplingParams`` (``crates/mach-model/src/sampling.rs:46-66``) and of
``ContinuousModel::add`` (``crates/mach-model/src/continuous.rs:715-723``): temperature, top_k,
top_p, seed, presence_penalty, frequency_penalty, max_new, eos, stop.

    python -m machserve_amd --model DIR --prompt-ids 1,2,3 --max-new 16
    python -m machserve_amd --random-config config.json --seed 0 --prompt-file prompts.txt
    python -m machserve_amd random-weights --config config.json --seed 0 --out DIR [--dtype f32|bf16|f16]
    python -m machserve_amd doctor
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile

from . import __version__


def _env(name: str, default=None):
    v = os.environ.get(name)
    return default if v in (None, "") else v


def _ids(text: str):
    return [int(t) for t in text.replace(",", " ").split()]


def doctor() -> int:
    """Environment and GPU report (``crates/mach-server/src/main.rs:246-300``)."""
    import torch
    from .kernels import build
    print(f"machserve_amd {__version__}")
    for k in ("MACH_MODEL", "MACH_DTYPE", "MACH_CAPACITY", "MACH_PREFILL_ROWS", "MACH_TPP", "MACH_MAX_SEQ"):
        print(f"  {k}={os.environ.get(k, '')}")
    print(f"  torch {torch.__version__}, hip {getattr(torch.version, 'hip', None)}")
    if torch.cuda.is_available():
        p = torch.cuda.get_device_properties(0)
        free, total = torch.cuda.mem_get_info(0)
        print(f"  GPU 0: {p.name} ({getattr(p, 'gcnArchName', '?')}), {p.multi_processor_count} CUs, "
              f"{total / 2**30:.0f} GiB ({free / 2**30:.0f} free)")
    else:
        print("  no GPU visible")
    try:
        print(f"  hipcc: {build._hipcc()}")
    except build.BuildError as e:
        print(f"  {e}")
    print(f"  libraries: {build._lib_dir()}")
    return 0


def random_weights(argv) -> int:
    """Write a model folder (config.json, model.safetensors) with random weights."""
    import torch
    from .weights import write_random_model
    ap = argparse.ArgumentParser(prog="machserve_amd random-weights", description=random_weights.__doc__)
    ap.add_argument("--config", required=True, help="config.json of the architecture")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--out", required=True, help="folder to write")
    ap.add_argument("--dtype", default="f32", choices=["f32", "bf16", "f16"], help="dtype the tensors are stored in")
    args = ap.parse_args(argv)
    with open(args.config) as f:
        raw = json.load(f)
    out = write_random_model(raw, args.seed, args.out, {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[args.dtype])
    print(out)
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] == "doctor":
        return doctor()
    if argv and argv[0] == "random-weights":
        return random_weights(argv[1:])
    ap = argparse.ArgumentParser(prog="machserve_amd", description=__doc__.split("\n\n")[0])
    ap.add_argument("--version", action="version", version=f"machserve_amd {__version__}")
    ap.add_argument("--model", default=_env("MACH_MODEL"), help="folder with config.json and model.safetensors")
    ap.add_argument("--random-config", help="config.json to build random weights from instead of --model")
    ap.add_argument("--weights-seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--dtype", default=_env("MACH_DTYPE", "bf16"), help="bf16 | f16 | f32 (MACH_DTYPE of the reference: f16 | f32)")
    ap.add_argument("--prompt-ids", action="append", default=[], help="token ids of one prompt, comma separated")
    ap.add_argument("--prompt-file", help="one prompt a line, token ids separated by spaces or commas")
    ap.add_argument("--max-new", type=int, default=16)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=0, help="sampling seed; 0 uses the request's id")
    ap.add_argument("--presence-penalty", type=float, default=0.0)
    ap.add_argument("--frequency-penalty", type=float, default=0.0)
    ap.add_argument("--top-logprobs", type=int, default=0, help="report this many most probable tokens per step (--json)")
    ap.add_argument("--eos", type=int, default=None)
    ap.add_argument("--stop", action="append", default=[], help="a stop sequence of token ids, comma separated")
    ap.add_argument("--capacity", type=int, default=int(_env("MACH_CAPACITY", 64)), help="requests running at once")
    ap.add_argument("--prefill-rows", type=int, default=int(_env("MACH_PREFILL_ROWS", 512)), help="tokens per step")
    ap.add_argument("--chunk-size", type=int, default=None, help="longest prompt portion of one request in a step")
    ap.add_argument("--tpp", type=int, default=int(_env("MACH_TPP", 64)), help="tokens per page")
    ap.add_argument("--num-pages", type=int, default=None, help="pages of the cache pool")
    ap.add_argument("--max-seq", type=int, default=int(_env("MACH_MAX_SEQ", 0)) or None,
                    help="longest request (prompt and generated); sizes the pool when --num-pages is absent")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--json", action="store_true", help="print one JSON object per prompt")
    args = ap.parse_args(argv)

    prompts = [_ids(p) for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [_ids(line) for line in f if line.strip()]
    if not prompts:
        ap.error("no prompt: give --prompt-ids or --prompt-file")
    if bool(args.model) == bool(args.random_config):
        ap.error("give exactly one of --model and --random-config")

    from .engine import Engine
    from .sampling import SamplingParams
    tmp = None
    model_dir = args.model
    if args.random_config:
        from .weights import write_random_model
        with open(args.random_config) as f:
            raw = json.load(f)
        tmp = tempfile.TemporaryDirectory(prefix="machserve_random_")
        model_dir = write_random_model(raw, args.weights_seed, tmp.name)
    tpp = args.tpp
    if args.num_pages is None:
        per_request = args.max_seq or max(len(p) for p in prompts) + args.max_new
        num_pages = min(len(prompts), args.capacity) * (-(-per_request // tpp))
    else:
        num_pages = args.num_pages
    engine = Engine.from_dir(model_dir, dtype=args.dtype, device=args.device, page_size=tpp, num_pages=num_pages,
                             capacity=args.capacity, max_batch_tokens=args.prefill_rows, chunk_size=args.chunk_size)
    ids = []
    for i, p in enumerate(prompts):
        params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                                seed=(args.seed + i) if args.seed else 0, presence_penalty=args.presence_penalty,
                                frequency_penalty=args.frequency_penalty, top_logprobs=args.top_logprobs)
        ids.append(engine.add(p, args.max_new, params, args.eos, [_ids(s) for s in args.stop]))
    done = engine.run()
    for i, p in zip(ids, prompts):
        r = done[i]
        if args.json:
            rec = {"prompt": p, "generated": r.generated, "finish_reason": r.finish_reason, "logprobs": r.logprobs}
            if args.top_logprobs:
                rec["top_logprobs"] = r.top_logprobs
            print(json.dumps(rec))
        else:
            print(" ".join(str(t) for t in r.generated))
    if tmp is not None:
        tmp.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
