"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--dtype bf16|f32]
                    [--shape 0.5b|1.5b|7b] [--batch B] [--context C] [--page-size P]

Default run: Qwen2.5-0.5B layer sizes with random weights (synthetic token ids), 8 requests
that each hold a 2,048-token context, K decode steps through the whole engine (scheduler,
step function, sampler).  One JSON line: ``value`` is decoded tokens a second at batch 8;
``prefill`` is one 2,048-token prompt in one step; ``roofline`` prices the decode step's
mandatory bytes (every weight once, the live requests' cache) against 8 TB/s;
``points`` holds decode at batch 1 and 64.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "f32": 157.3e12}
# the reference's own numbers for this model on its hardware (RX 7900 XTX, fp16)
REF_DECODE_B64_CTX2048 = 4777.0   # README.md:15, docs/benchmark-protocol.md:74-75
REF_PREFILL_2048 = 2048 / 0.289   # README.md:18

QWEN25_05B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_size": 896, "num_hidden_layers": 24,
    "num_attention_heads": 14, "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936,
    "max_position_embeddings": 32768, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "tie_word_embeddings": True,
    "hidden_act": "silu", "use_sliding_window": False,
}


# the two larger configurations of the same architecture (random weights, same distribution)
QWEN25_15B = dict(QWEN25_05B, hidden_size=1536, num_hidden_layers=28, num_attention_heads=12, num_key_value_heads=2,
                  intermediate_size=8960)
QWEN25_7B = dict(QWEN25_05B, hidden_size=3584, num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4,
                 intermediate_size=18944, vocab_size=152064, tie_word_embeddings=False)
SHAPES = {"0.5b": ("Qwen2.5-0.5B", QWEN25_05B), "1.5b": ("Qwen2.5-1.5B", QWEN25_15B), "7b": ("Qwen2.5-7B", QWEN25_7B)}


def model_numbers(cfg, elem_bytes):
    d, L, H, KV, hd = cfg.hidden_size, cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    I, V = cfg.intermediate_size, cfg.vocab_size
    per_layer = (H * hd + 2 * KV * hd) * d + d * H * hd + 3 * I * d
    head = V * d
    weight_bytes = (L * per_layer + head) * elem_bytes + (L * (2 * d + (H + 2 * KV) * hd) + d) * 4
    kv_bytes_per_token = L * 2 * KV * hd * elem_bytes
    return {"per_layer": per_layer, "head": head, "weight_bytes": weight_bytes, "kv_bytes_per_token": kv_bytes_per_token}


def prefill_flops(cfg, T):
    n = model_numbers(cfg, 2)
    gemm = 2.0 * T * cfg.num_hidden_layers * n["per_layer"] + 2.0 * n["head"]
    attn = cfg.num_hidden_layers * 4.0 * cfg.num_attention_heads * cfg.head_dim * (T * (T + 1) / 2)
    return gemm + attn


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (named in config)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f32"])
    ap.add_argument("--shape", default="0.5b", choices=sorted(SHAPES), help="layer sizes (default: the 0.5B configuration)")
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    ap.add_argument("--sync-steps", action="store_true", help="wait for each decode step's tokens before the next is launched")
    ap.add_argument("--prefill-only", action="store_true", help="time the 2,048-token prefill alone (for profiles)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import Engine, load_model
    from machserve_amd.sampling import SamplingParams
    from machserve_amd.weights import random_tensor_dict

    shape_name, shape = SHAPES[args.shape]
    raw = dict(shape)
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    cfg = config_from_dict(raw)
    dt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    tensors = random_tensor_dict(cfg, 0, dt, device="cuda:0")
    ctx, page = args.context, args.page_size
    gen = torch.Generator().manual_seed(1)

    def prompts(n, length):
        return [torch.randint(0, cfg.vocab_size, (length,), generator=gen).tolist() for _ in range(n)]

    def make_engine(batch, budget):
        per_req = -(-(ctx + args.warmup + args.steps + 2 * batch + 96) // page)
        lm = load_model(config=cfg, tensors=tensors, dtype=dt, page_size=page, num_pages=batch * per_req + 4,
                        max_requests=batch)
        return Engine(lm, max_batch_tokens=budget, max_running=batch)

    def decode_run(batch):
        eng = make_engine(batch, 4096)
        for p in prompts(batch, ctx):
            eng.add(p, args.warmup + args.steps + 2 * batch + 88, SamplingParams())  # early ones decode while later ones prefill
        while any(not r.decoding for r in eng.scheduler.running) or eng.scheduler.waiting:
            eng.step()
        # the engine's own loop (Engine.run): a step is launched while the tokens of the step before
        # are on their way to the host, so the tokens a call returns are those of the launch before it
        step = eng.step if args.sync_steps else eng.step_pipelined
        # the engine captures a decode step into a graph once its shape has come a number of times:
        # that happens before the warm-up, not in the timed steps
        for _ in range(eng.loaded.step.DECODE_CAPTURE_AFTER + 2):
            step()
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        before, seen = eng.steps, 0
        t0 = time.perf_counter()
        for _ in range(args.steps):
            em, _ = step()
            seen += len(em)
        torch.cuda.synchronize()
        dt_s = time.perf_counter() - t0
        assert eng.steps - before == args.steps, "exactly the timed steps ran on the device"
        assert batch * (args.steps - 1) <= seen <= batch * args.steps  # the first call may have had nothing before it
        del eng
        torch.cuda.empty_cache()
        return batch * args.steps / dt_s, dt_s / args.steps * 1e3

    def prefill_run():
        eng = make_engine(1, ctx)
        times = []
        for rep in range(4):
            eng.add(prompts(1, ctx)[0], 1, SamplingParams())
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            em, done = eng.step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            assert len(em) == 1 and len(done) == 1
        del eng
        torch.cuda.empty_cache()
        return min(times[1:])

    nums = model_numbers(cfg, dt.itemsize)
    if args.prefill_only:
        t = prefill_run()
        print(json.dumps({"prefill": {"value": round(ctx / t, 1), "tokens": ctx, "ms": round(t * 1e3, 3),
                                      "frac": round(prefill_flops(cfg, ctx) / t / PEAK_FLOPS[args.dtype], 4)}}))
        return 0
    tok_s, ms = decode_run(args.batch)
    step_bytes = nums["weight_bytes"] + args.batch * (ctx + args.warmup + args.steps / 2) * nums["kv_bytes_per_token"]
    achieved = step_bytes / (ms * 1e-3) / 1e9
    out = {
        "metric": f"decode tok/s at batch {args.batch}, {ctx}-token contexts ({shape_name} shape)",
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0,0.02) seed 0, uniform random token ids",
        "config": {
            "model": f"{shape_name} shape (Qwen2ForCausalLM)", "global_batch": args.batch, "seq_len": ctx,
            "parallelism": "single GPU", "layers": cfg.num_hidden_layers, "layers_of_configuration": full_layers,
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "tied_head": bool(cfg.tie_word_embeddings), "rope_theta": cfg.rope_theta, "rms_eps": cfg.rms_norm_eps,
            "page_size": page, "prefill_tokens": ctx, "sampling": "greedy",
            "stepping": "one at a time" if args.sync_steps else "launched one step ahead",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
    }
    if not args.no_points:
        t = prefill_run()
        fl = prefill_flops(cfg, ctx)
        out["prefill"] = {"value": round(ctx / t, 1), "tokens": ctx, "ms": round(t * 1e3, 3),
                          "frac": round(fl / t / PEAK_FLOPS[args.dtype], 4)}
        b1, _ = decode_run(1)
        b64, _ = decode_run(64)
        out["points"] = {"decode_b1": round(b1, 1), "decode_b64": round(b64, 1)}
        if args.dtype == "bf16" and cfg.num_hidden_layers == full_layers and args.shape == "0.5b" and ctx == 2048:
            out["vs_reference"] = {"decode_b64_ctx2048": round(b64 / REF_DECODE_B64_CTX2048, 2),
                                   "prefill_2048": round(ctx / t / REF_PREFILL_2048, 2)}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
