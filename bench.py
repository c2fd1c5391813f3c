"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--dtype bf16|f32]
                    [--shape 0.5b|1.5b|7b] [--batch B] [--context C] [--page-size P]
                    [--no-points] [--no-kernels] [--more-shapes]

Default run: Qwen2.5-0.5B layer sizes with random weights (synthetic token ids), 8 requests
that each hold a 2,048-token context, K decode steps through the whole engine (scheduler,
step function, sampler), timed three times in a row; the median window is reported.  One JSON
line: ``value`` is decoded tokens a second at batch 8; ``prefill`` is one 2,048-token prompt in
one step; ``roofline`` prices the decode step's mandatory bytes (every weight once, the live
requests' cache) against 8 TB/s; ``points`` holds decode at batch 1 and 64, decode at longer
contexts and a longer prefill (``points_detail``: their times and fractions of the published
peak); ``launches_per_step`` counts the kernels of a decode step; ``measured_peaks`` is what the
box itself gives a device-to-device copy and a loop of matrix instructions; ``kernels`` breaks
the decode step and the prefill down by kind of kernel (time a step, GB/s or TFLOP/s, fraction
of the published and of the measured peak), from a second run of the same work under
``rocprofv3 --kernel-trace`` whose dispatches are matched, in order, with the operations that
the step issues.

Method of the reference: time per step over a fixed number of steps after a warm-up
(``crates/mach-model/examples/lctx_bench.rs:64-89``, ``docs/benchmark-protocol.md:43-75``).
"""
from __future__ import annotations

import argparse
import csv
import glob
import json
import os
import shutil
import statistics
import subprocess
import sys
import tempfile
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "f16": 2.5e15, "f32": 157.3e12}
# the reference's own numbers for this model on its hardware (RX 7900 XTX, fp16)
REF_DECODE_B64_CTX2048 = 4777.0   # README.md:15, docs/benchmark-protocol.md:74-75
REF_PREFILL_2048 = 2048 / 0.289   # README.md:18
REF_DECODE_B256_SHORT = 29273.0   # docs/roadmap.md:324-325 (short contexts)
REF_DECODE_B512_SHORT = 35251.0   # the same sweep's last entry

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


# ------------------------------------------------------------------------------------ the operations of a step, by kind

PRODUCT_OPS = {  # name -> positions of (rows operand, weight) among the arguments
    "linear_split": (0, 1), "linear": (0, 1), "linear_residual": (0, 1), "linear_residual_prenorm": (0, 1),
    "linear_swiglu": (0, 1), "linear_swiglu_scaled": (0, 3), "linear_split_normed": (0, 4), "linear_swiglu_normed": (0, 4),
    "linear_qkv_rope": (0, 1),
}
OTHER_OPS = {"embed": "embedding", "rmsnorm": "norm", "add_partials": "norm", "rope_kv_write": "rotation and cache write",
             "rope_table": "rotation and cache write",
             "paged_attention": "attention", "decode_attention_fused": "attention", "decode_attention": "attention",
             "sample": "sampling", "sample_packed": "sampling", "top_logprobs": "sampling", "logit_edit": "sampling"}


class Recorder:
    """Wraps the kernel boundary's methods: while ``on()`` says so, every outermost call is listed with its kind,
    the kernels it launched, and for a matrix product the bytes of its weight and its floating-point operations."""

    def __init__(self, ops, vocab, on):
        self.ops, self.calls, self.depth, self.on = ops, [], 0, on
        for name in list(PRODUCT_OPS) + list(OTHER_OPS):
            setattr(ops, name, self._wrap(name, getattr(ops, name), vocab))

    def _wrap(self, name, inner, vocab):
        def call(*a, **kw):
            if self.depth or not self.on():
                return inner(*a, **kw)
            self.depth += 1
            before = self.ops.launch_count()
            try:
                out = inner(*a, **kw)
            finally:
                self.depth -= 1
            launched = self.ops.launch_count() - before
            kind, nbytes, flops = OTHER_OPS.get(name), 0, 0
            if name in PRODUCT_OPS:
                rows, w = a[PRODUCT_OPS[name][0]], a[PRODUCT_OPS[name][1]]
                kind = "head" if w.shape[0] >= vocab else "products"
                nbytes, flops = w.numel() * w.element_size(), 2 * rows.shape[0] * w.numel()
            self.calls.append([kind, launched, nbytes, flops])
            return out
        return call


def trace_rows(folder):
    """(start, end, name) of every dispatch of the engine's own kernels in a rocprofv3 kernel trace, in order."""
    rows = []
    for path in glob.glob(os.path.join(folder, "**", "*kernel_trace.csv"), recursive=True):
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                if "ms::" in r["Kernel_Name"] or "_ZN2ms" in r["Kernel_Name"]:  # (some names come without being demangled)
                    rows.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), r["Kernel_Name"]))
    rows.sort()
    return rows


def by_name(rows, n):
    """The dispatches ``rows[-n:]`` by kernel name: (name, calls, mean microseconds, total microseconds), longest total first."""
    names = {}
    for start, end, name in rows[-n:]:
        k = names.setdefault(name, [0, 0.0])
        k[0] += 1
        k[1] += (end - start) / 1e3
    return sorted(((nm, c, t / c, t) for nm, (c, t) in names.items()), key=lambda r: -r[3])


def write_summary(path, title, command, kinds, names, n_steps, work_of=None):
    """A short text summary of one traced run: what it ran, the kinds of kernels, the kernels by name (with the rate of
    those whose bytes or operations ``work_of`` knows: name -> (amount over the listed calls, unit))."""
    lines = [f"# {title}", "", "Command (on an MI355X, from the repository root; the summary is written by the command itself):", "",
             f"    {command}", "",
             "The work is run a second time under `rocprofv3 --kernel-trace`; the dispatches of the last steps are matched, in order, with",
             "the operations one step issues.  Times are the kernels' own durations as the profiler reports them.", "",
             "| kind of kernel | launches a step | us a step | rate | of the published peak | of what the box gives |", "|---|---|---|---|---|---|"]
    for kind, r in kinds.items():
        if kind == "all" or kind.startswith("_") or not isinstance(r, dict):
            continue
        rate = f"{r['rate']} {r['unit']}" if "rate" in r else ""
        lines.append(f"| {kind} | {r['launches']} | {r['us']} | {rate} | {r.get('frac', '')} | {r.get('frac_of_measured', '')} |")
    if isinstance(kinds.get("all"), dict):
        a = kinds["all"]
        lines += ["", f"All: {a['launches']} launches a step, {a['us_in_kernels']} us inside kernels, {a['us_first_to_last']} us from the first "
                      f"kernel's start to the last one's end under the profiler (which slows the replay of a captured step)."]
    lines += ["", f"| kernel | calls in {n_steps} step{'s' if n_steps != 1 else ''} | mean us | total us | rate |", "|---|---|---|---|---|"]
    for nm, c, mean, total in names[:14]:
        rate = ""
        if work_of and nm in work_of and total > 0:
            amount, unit = work_of[nm]
            rate = f"{amount / (total * 1e-6) / (1e9 if unit == 'GB/s' else 1e12):.0f} {unit}"
        lines.append(f"| `{nm[:110]}` | {c} | {mean:.2f} | {total:.1f} | {rate} |")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def account(calls, rows, n_steps, peak_of, measured_of, extra):
    """Per kind of kernel: launches and microseconds a step, and with the kind's bytes or operations its rate and the
    fractions of the published and of the measured peak.  ``calls`` lists one step's operations in order; ``rows``
    ends with the dispatches of ``n_steps`` such steps."""
    per_launch = [c for c in calls for _ in range(c[1])]
    L = len(per_launch)
    if L == 0 or len(rows) < n_steps * L:
        return {"error": f"{len(rows)} traced dispatches for {n_steps} steps of {L} launches"}
    rows = rows[-n_steps * L:]
    kinds = {}
    # what the dispatches of a kernel name moved or computed, where an operation is one launch (a product) or its
    # work is given for the kind (attention)
    work_of, kind_us = {}, {}
    for i, (start, end, name) in enumerate(rows):
        call = per_launch[i % L]
        k = kinds.setdefault(call[0], {"launches": 0, "us": 0.0})
        k["us"] += (end - start) / 1e3 / n_steps
        unit = peak_of.get(call[0])
        if unit and call[1] == 1 and call[0] not in extra:
            w = work_of.setdefault(name, [0.0, unit])
            w[0] += call[2] if unit == "GB/s" else call[3]
        elif unit and call[0] in extra:
            kind_us.setdefault(call[0], {}).setdefault(name, [0.0])[0] += (end - start) / 1e3
    for c in calls:
        k = kinds.setdefault(c[0], {"launches": 0, "us": 0.0})
        k["launches"] += c[1]
        k["bytes"] = k.get("bytes", 0) + c[2]
        k["flops"] = k.get("flops", 0) + c[3]
    for name, (nbytes, flops) in extra.items():
        if name in kinds:
            kinds[name]["bytes"], kinds[name]["flops"] = nbytes, flops
    out = {}
    for name, k in kinds.items():
        rec = {"launches": k["launches"], "us": round(k["us"], 2)}
        unit = peak_of.get(name)
        work = k.get("bytes", 0) if unit == "GB/s" else k.get("flops", 0)
        if unit and work and k["us"] > 0:
            rate = work / (k["us"] * 1e-6) / (1e9 if unit == "GB/s" else 1e12)
            peak = PEAK_HBM_GBS if unit == "GB/s" else peak_of["flops_peak"] / 1e12
            rec.update({"rate": round(rate, 1), "unit": unit if unit == "GB/s" else "TFLOP/s", "frac": round(rate / peak, 4)})
            if measured_of.get(unit):
                rec["frac_of_measured"] = round(rate / measured_of[unit], 4)
        out[name] = rec
    span = sum((rows[(s + 1) * L - 1][1] - rows[s * L][0]) for s in range(n_steps)) / 1e3 / n_steps
    busy = sum(k["us"] for k in kinds.values())
    out["all"] = {"launches": L, "us_in_kernels": round(busy, 2), "us_first_to_last": round(span, 2),
                  "us_between_kernels": round(span - busy, 2)}
    for kind, per_name in kind_us.items():
        unit = peak_of[kind]
        amount = (extra[kind][0] if unit == "GB/s" else extra[kind][1]) * n_steps
        main = max(per_name, key=lambda n: per_name[n][0])  # the kind's work is its main kernel's (a merge moves next to nothing)
        work_of[main] = [amount, unit]
    out["_work_of"] = {k: (v[0], "GB/s" if v[1] == "GB/s" else "TFLOP/s") for k, v in work_of.items()}
    return out


def measured_peaks(dtype_name):
    """What the box gives: a device-to-device copy of 1 GiB (bytes read plus written over the time) and a loop of
    nothing but matrix instructions of the run's element type."""
    import ctypes
    import torch
    from machserve_amd.kernels import build
    out = {}
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0")
    dst = torch.empty_like(src)
    best = 1e9
    for _ in range(5):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        dst.copy_(src)
        b.record()
        b.synchronize()
        best = min(best, a.elapsed_time(b))
    out["copy_GBs"] = round(2 * (1 << 30) / (best * 1e-3) / 1e9, 1)
    del src, dst
    lib = ctypes.CDLL(build_probe(dtype_name))
    blocks, iters = 4096, 2048 if dtype_name == "bf16" else 1024
    buf = torch.empty(blocks * 256, dtype=torch.float32, device="cuda:0")
    flops = ctypes.c_double(0.0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    best = 1e9
    for _ in range(4):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        if lib.ms_probe_mfma(ctypes.c_void_p(buf.data_ptr()), blocks, iters, ctypes.byref(flops), stream) != 0:
            return out
        b.record()
        b.synchronize()
        best = min(best, a.elapsed_time(b))
    out["mfma_TFLOPs"] = round(flops.value / (best * 1e-3) / 1e12, 1)
    return out


def build_probe(dtype_name, force=False):
    """The matrix-core measurement beside this file, compiled into a library of its own (this benchmark's, not the
    package's: nothing on the product path loads it)."""
    from machserve_amd.kernels import build
    here = os.path.dirname(os.path.abspath(__file__))
    return build.ensure_extra_library("bench_mfma_probe", dtype_name, os.path.join(here, "bench_mfma_probe.hip"), force)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (named in config)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16", "f32"])
    ap.add_argument("--shape", default="0.5b", choices=sorted(SHAPES), help="layer sizes (default: the 0.5B configuration)")
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--no-points", action="store_true", help="skip the further points and the prefill")
    ap.add_argument("--no-kernels", action="store_true", help="skip the break-down by kind of kernel (a second run under rocprofv3)")
    ap.add_argument("--more-shapes", action="store_true", help="further decode and prefill points of the 1.5B and 7B layer sizes")
    ap.add_argument("--fewer-points", action="store_true", help="skip the points in other precisions, of other layer sizes and of the first token")
    ap.add_argument("--sync-steps", action="store_true", help="wait for each decode step's tokens before the next is launched")
    ap.add_argument("--prefill-only", action="store_true", help="time the prefill alone (for profiles)")
    ap.add_argument("--prefill-tokens", type=int, default=None, help="tokens of the prefill (default: the context)")
    ap.add_argument("--profile-out", default=None, help="folder that receives a summary of the traced runs, one text file for the decode "
                    "step and one for the prefill (kinds of kernels, and the kernels by name)")
    ap.add_argument("--record-calls", default=None, help=argparse.SUPPRESS)  # file that receives one step's operations (the traced run)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import Engine, load_model
    from machserve_amd.sampling import SamplingParams
    from machserve_amd.weights import random_tensor_dict

    DT = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}
    dt = DT[args.dtype]
    gen = torch.Generator().manual_seed(1)
    models = {}

    def model_of(shape, dtn=None):
        dtn = dtn or args.dtype
        if (shape, dtn) not in models:
            raw = dict(SHAPES[shape][1])
            full = raw["num_hidden_layers"]
            if args.layers and shape == args.shape:
                raw["num_hidden_layers"] = args.layers
            cfg = config_from_dict(raw)
            models.clear()  # one model's weights at a time
            torch.cuda.empty_cache()
            models[(shape, dtn)] = (cfg, random_tensor_dict(cfg, 0, DT[dtn], device="cuda:0"), full)
        return models[(shape, dtn)]

    def prompts(cfg, n, length):
        return [torch.randint(0, cfg.vocab_size, (length,), generator=gen).tolist() for _ in range(n)]

    recording = [False]
    recorders = []

    def head_start(batch, ctx, budget):
        """Tokens that the first request may decode while the last one's prompt is still being fed (a step takes every
        decoding request's token and ``budget`` tokens in all): what a request is given beyond the timed steps."""
        return max(2 * batch + 88, -(-batch * ctx // max(budget - batch, 1)) + batch + 24)

    def make_engine(shape, batch, budget, ctx, windows=1, dtn=None, page=None):
        cfg, tensors, _ = model_of(shape, dtn)
        page = page or args.page_size
        per_req = -(-(ctx + args.warmup + windows * args.steps + head_start(batch, ctx, budget) + 8) // page)
        lm = load_model(config=cfg, tensors=tensors, dtype=DT[dtn or args.dtype], page_size=page, num_pages=batch * per_req + 4,
                        max_requests=batch)
        if args.record_calls and not recorders:
            recorders.append(Recorder(lm.rt.ops, cfg.vocab_size, lambda: recording[0]))
        return Engine(lm, max_batch_tokens=budget, max_running=batch)

    def decode_run(shape, batch, ctx, windows=3, dtn=None, page=None):
        """(tokens a second, milliseconds a step) of the median of ``windows`` timed runs of ``--steps`` decode steps."""
        cfg = model_of(shape, dtn)[0]
        eng = make_engine(shape, batch, 4096, ctx, windows, dtn, page)
        for p in prompts(cfg, batch, ctx):
            eng.add(p, args.warmup + windows * args.steps + head_start(batch, ctx, 4096), SamplingParams())  # early ones decode while later ones prefill
        while any(not r.decoding for r in eng.scheduler.running) or eng.scheduler.waiting:
            eng.step()
        # the engine's own loop (Engine.run): a step is launched while the tokens of the step before
        # are on their way to the host, so the tokens a call returns are those of the launch before it
        step = eng.step if args.sync_steps else eng.step_pipelined
        # the engine captures a decode step into a graph once its shape has come a number of times:
        # that happens before the warm-up, not in the timed steps
        recording[0] = bool(args.record_calls)  # the capture issues the step's operations once: they are listed then
        for _ in range(eng.loaded.step.DECODE_CAPTURE_AFTER + 2):
            step()
        for _ in range(args.warmup):
            step()
        times = []
        for _ in range(windows):
            torch.cuda.synchronize()
            before, seen = eng.steps, 0
            t0 = time.perf_counter()
            for _ in range(args.steps):
                em, _ = step()
                seen += len(em)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            assert eng.steps - before == args.steps, "exactly the timed steps ran on the device"
            assert batch * (args.steps - 1) <= seen <= batch * args.steps  # the first call may have had nothing before it
        recording[0] = False
        del eng
        torch.cuda.empty_cache()
        dt_s = statistics.median(times)
        return batch * args.steps / dt_s, dt_s / args.steps * 1e3

    def prefill_run(shape, tokens, dtn=None):
        cfg = model_of(shape, dtn)[0]
        eng = make_engine(shape, 1, tokens, tokens, 1, dtn)
        times = []
        # a step of a size that keeps coming is captured after a few sightings and then replayed, as in serving: the first
        # ones are launched kernel by kernel, one captures, the last three are timed
        for rep in range(eng.loaded.step.FILLED_CAPTURE_AFTER + 4):
            eng.add(prompts(cfg, 1, tokens)[0], 1, SamplingParams())
            torch.cuda.synchronize()
            recording[0] = bool(args.record_calls)  # the capture issues the step's operations once: they are listed then
            t0 = time.perf_counter()
            em, done = eng.step()
            torch.cuda.synchronize()
            recording[0] = False
            times.append(time.perf_counter() - t0)
            assert len(em) == 1 and len(done) == 1
        del eng
        torch.cuda.empty_cache()
        return min(times[-3:])

    def decode_bytes(cfg, batch, ctx, windows, dtn=None):
        nums = model_numbers(cfg, DT[dtn or args.dtype].itemsize)
        mean_ctx = ctx + args.warmup + windows * args.steps / 2
        return nums["weight_bytes"] + batch * mean_ctx * nums["kv_bytes_per_token"]

    def decode_point(shape, batch, ctx, dtn=None, page=None):
        tok_s, ms = decode_run(shape, batch, ctx, 3, dtn, page)
        rate = decode_bytes(model_of(shape, dtn)[0], batch, ctx, 3, dtn) / (ms * 1e-3) / 1e9
        return tok_s, {"ms": round(ms, 4), "GBs": round(rate, 1), "frac": round(rate / PEAK_HBM_GBS, 4)}

    def prefill_point(shape, tokens, dtn=None):
        t = prefill_run(shape, tokens, dtn)
        fl = prefill_flops(model_of(shape, dtn)[0], tokens)
        return tokens / t, {"ms": round(t * 1e3, 3), "TFLOPs": round(fl / t / 1e12, 1),
                            "frac": round(fl / t / PEAK_FLOPS[dtn or args.dtype], 4)}

    def first_token_points(shape, lengths):
        """Time to the first token of one prompt, from ``add`` to its sampled token on the host, for prompts of
        lengths that the engine has not seen: the steps of the sizes that prompts are filled up to (every 64
        tokens up to 512) were captured before, by ``Engine.warm_up``, with other tokens."""
        cfg = model_of(shape)[0]
        eng = make_engine(shape, 2, 1024, 1024)
        eng.warm_up(range(64, 513, 64))
        out = {}
        for n in lengths:
            times = []
            for rep in range(3):   # other tokens each time; the first is the cold one of this length
                eng.add(prompts(cfg, 1, n)[0], 1, SamplingParams())
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                em, done = eng.step()
                times.append(time.perf_counter() - t0)
                assert len(em) == 1 and len(done) == 1
            fl = prefill_flops(cfg, n)
            out[n] = (n / times[0], {"ms": round(times[0] * 1e3, 3), "ms_again": round(min(times[1:]) * 1e3, 3),
                                     "TFLOPs": round(fl / times[0] / 1e12, 1), "frac": round(fl / times[0] / PEAK_FLOPS[args.dtype], 4)})
        del eng
        torch.cuda.empty_cache()
        return out

    def mixed_load_point(shape, n_requests=256, running=64, budget=2048, arrive=4):
        """The whole engine under a load as a server has it: requests of 64 to 640 prompt tokens and 32 to 256 new tokens,
        ``arrive`` of them a step, at most ``running`` at a time, prompts fed in portions beside the decoding requests
        under a budget of ``budget`` tokens a step, to the end.  Tokens a second, prompt and generated together, from
        the first arrival to the last token on the host; the sizes that steps are filled up to were captured before
        (``Engine.warm_up``), the decode steps' shapes are captured as they come."""
        import random
        cfg, tensors, _ = model_of(shape)
        lm = load_model(config=cfg, tensors=tensors, dtype=DT[args.dtype], page_size=args.page_size, max_tokens=running * 1024,
                        max_requests=running)
        eng = Engine(lm, max_batch_tokens=budget, max_running=running)
        eng.warm_up(range(64, budget + 1, 64))
        rng = random.Random(0)
        reqs = [([rng.randrange(cfg.vocab_size) for _ in range(rng.randint(64, 640))], rng.randint(32, 256)) for _ in range(n_requests)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        added = produced = steps = 0
        while added < n_requests or eng.has_work():
            for p, m in reqs[added:added + arrive]:
                eng.add(p, m, SamplingParams())
            added = min(n_requests, added + arrive)
            em, _ = eng.step_pipelined()
            produced += len(em)
            steps += 1
        torch.cuda.synchronize()
        dt_s = time.perf_counter() - t0
        prompt_tokens = sum(len(p) for p, _ in reqs)
        assert produced == sum(m for _, m in reqs), "every request ran to its last token"
        del eng, lm
        torch.cuda.empty_cache()
        return (prompt_tokens + produced) / dt_s, {"s": round(dt_s, 3), "requests": n_requests, "prompt_tokens": prompt_tokens,
                                                   "generated": produced, "generated_tok_s": round(produced / dt_s, 1),
                                                   "steps": steps, "ms_per_step": round(dt_s / steps * 1e3, 3)}

    shape_name = SHAPES[args.shape][0]
    cfg, _, full_layers = model_of(args.shape)
    ctx = args.context
    prefill_tokens = args.prefill_tokens or ctx

    def save_calls(kind):
        """The traced run's list of one step's operations: the last time the model's operations were issued (launched, or
        recorded into a graph), and the sampling after it (inside the graph for decoding, after the step for a prompt)."""
        calls = recorders[0].calls if recorders else []
        starts = [i for i, c in enumerate(calls) if c[0] == "embedding"]
        if kind == "decode":  # the capture ran the step's operations once under recording: the last such run
            ends = [i for i, c in enumerate(calls) if c[0] == "sampling"]
            if ends and starts:
                first = max(s for s in starts if s < ends[-1])
                calls = calls[first:ends[-1] + 1]
        elif starts:
            first = last = starts[-1]
            while last < len(calls) and calls[last][0] != "sampling":
                last += 1
            calls = calls[first:last + 1]  # with the one sampling call that follows the step (later steps, replayed, list only theirs)
        with open(args.record_calls, "w") as f:
            json.dump(calls, f)

    if args.prefill_only:
        tok_s, rec = prefill_point(args.shape, prefill_tokens)
        if args.record_calls:
            save_calls("prefill")
        print(json.dumps({"prefill": {"value": round(tok_s, 1), "tokens": prefill_tokens, **rec}}))
        return 0
    if args.record_calls:  # the traced run: one window, nothing else
        decode_run(args.shape, args.batch, ctx, windows=1)
        save_calls("decode")
        return 0

    tok_s, ms = decode_run(args.shape, args.batch, ctx)
    achieved = decode_bytes(cfg, args.batch, ctx, 3) / (ms * 1e-3) / 1e9
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
            "page_size": args.page_size, "prefill_tokens": prefill_tokens, "sampling": "greedy",
            "stepping": "one at a time" if args.sync_steps else "launched one step ahead",
        },
        "timed": "median of three windows of `steps` steps",
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
    }
    peaks = measured_peaks(args.dtype)
    out["measured_peaks"] = peaks
    if peaks.get("copy_GBs"):
        out["roofline"]["frac_of_measured_copy"] = round(achieved / peaks["copy_GBs"], 4)
    if not args.no_points:
        p_tok_s, p = prefill_point(args.shape, prefill_tokens)
        out["prefill"] = {"value": round(p_tok_s, 1), "tokens": prefill_tokens, "ms": p["ms"], "frac": p["frac"]}
        points, detail = {}, {}
        for name, batch, c in (("decode_b1", 1, ctx), ("decode_b64", 64, ctx), ("decode_b8_ctx8192", 8, 8192),
                               ("decode_b8_ctx32000", 8, 32000)):
            if c + 4 * args.steps + 300 > cfg.max_position_embeddings:
                continue
            v, detail[name] = decode_point(args.shape, batch, c)
            points[name] = round(v, 1)
        v, detail["prefill_8192"] = prefill_point(args.shape, 8192)
        points["prefill_8192"] = round(v, 1)
        if args.dtype == "bf16" and cfg.num_hidden_layers == full_layers and args.shape == "0.5b" and ctx == 2048:
            out["vs_reference"] = {"decode_b64_ctx2048": round(points["decode_b64"] / REF_DECODE_B64_CTX2048, 2),
                                   "prefill_2048": round(p_tok_s / REF_PREFILL_2048, 2)}
        if args.shape == "0.5b" and args.dtype == "bf16" and cfg.num_hidden_layers == full_layers and not args.fewer_points:
            # the first token of a prompt of a length not seen before (the reference quotes 512 tokens, docs/roadmap.md:260-261)
            for n, (v, d) in first_token_points(args.shape, (128, 500, 512)).items():
                points[f"first_token_{n}"], detail[f"first_token_{n}"] = round(v, 1), d
            # the engine whole: arrivals, portions of prompts beside decoding requests, ends
            v, detail["mixed_load_256_requests"] = mixed_load_point(args.shape)
            points["mixed_load_256_requests"] = round(v, 1)
            # many requests at short contexts, as the reference's own sweep over the batch has them (docs/roadmap.md:324-325)
            v, detail["decode_b256_ctx512"] = decode_point(args.shape, 256, 512)
            points["decode_b256_ctx512"] = round(v, 1)
            if "vs_reference" in out:
                out["vs_reference"]["decode_b256_short_contexts"] = round(v / REF_DECODE_B256_SHORT, 2)
            v, detail["decode_b512_ctx512"] = decode_point(args.shape, 512, 512)
            points["decode_b512_ctx512"] = round(v, 1)
            if "vs_reference" in out:
                out["vs_reference"]["decode_b512_short_contexts"] = round(v / REF_DECODE_B512_SHORT, 2)
            # the same configuration in the reference's own fast precision and in true 32-bit
            for dtn in ("f16", "f32"):
                v, detail[f"{dtn}_decode_b8"] = decode_point(args.shape, args.batch, ctx, dtn)
                points[f"{dtn}_decode_b8"] = round(v, 1)
                v, detail[f"{dtn}_prefill_2048"] = prefill_point(args.shape, 2048, dtn)
                points[f"{dtn}_prefill_2048"] = round(v, 1)
            # the two larger configurations of the same architecture: 1.5B, eight requests of 512 tokens decoding with pages
            # of 16 tokens; 7B, 64 requests at 2,048-token contexts and one 2,048-token prompt
            runs = {"1.5b": [("decode_b8", 8, 512, 16)], "7b": [("decode_b64", 64, 2048, None)]}
            if args.more_shapes:
                runs["1.5b"].append(("decode_b64", 64, 2048, None))
                runs["7b"].insert(0, ("decode_b1", 1, 2048, None))
            for shape, rs in runs.items():
                for name, batch, c, pg in rs:
                    v, detail[f"{shape}_{name}_ctx{c}"] = decode_point(shape, batch, c, None, pg)
                    points[f"{shape}_{name}_ctx{c}"] = round(v, 1)
                if shape == "7b" or args.more_shapes:
                    v, detail[f"{shape}_prefill_2048"] = prefill_point(shape, 2048)
                    points[f"{shape}_prefill_2048"] = round(v, 1)
        out["points"], out["points_detail"] = points, detail
    models.clear()
    torch.cuda.empty_cache()
    if not args.no_kernels:
        out["kernels"] = kernels_by_kind(args, cfg, dt, peaks, ctx, prefill_tokens)
        if isinstance(out["kernels"].get("decode"), dict) and "all" in out["kernels"]["decode"]:
            out["launches_per_step"] = out["kernels"]["decode"]["all"]["launches"]
    print(json.dumps(out))
    return 0


def kernels_by_kind(args, cfg, dt, peaks, ctx, prefill_tokens):
    """The decode step and the prefill again under ``rocprofv3 --kernel-trace``, in processes of their own; their
    dispatches are matched in order with the operations that the traced run lists for one step."""
    prof = shutil.which("rocprofv3") or ("/opt/rocm/bin/rocprofv3" if os.path.exists("/opt/rocm/bin/rocprofv3") else None)
    if prof is None:
        return {"error": "rocprofv3 not found"}
    me = os.path.abspath(__file__)
    base = [sys.executable, me, "--steps", str(args.steps), "--warmup", str(args.warmup), "--batch", str(args.batch), "--context", str(ctx),
            "--dtype", args.dtype, "--shape", args.shape, "--page-size", str(args.page_size)] + (["--layers", str(args.layers)] if args.layers else [])
    nums = model_numbers(cfg, dt.itemsize)
    measured = {"GB/s": peaks.get("copy_GBs"), "TFLOP/s": peaks.get("mfma_TFLOPs")}
    out = {}
    env = dict(os.environ, TMPDIR=tempfile.gettempdir())
    for kind in ("decode", "prefill"):
        with tempfile.TemporaryDirectory() as tmp:
            calls_file = os.path.join(tmp, "calls.json")
            cmd = [prof, "--kernel-trace", "--output-format", "csv", "-d", os.path.join(tmp, "trace"), "--"] + base + ["--record-calls", calls_file]
            if kind == "prefill":
                cmd += ["--prefill-only", "--prefill-tokens", str(prefill_tokens)]
            try:
                r = subprocess.run(cmd, capture_output=True, text=True, timeout=150, cwd=tmp, env=env)
                if r.returncode != 0 or not os.path.exists(calls_file):
                    out[kind] = {"error": f"the traced run ended with {r.returncode}: {r.stderr[-300:]}"}
                    continue
                with open(calls_file) as f:
                    calls = json.load(f)
                rows = trace_rows(os.path.join(tmp, "trace"))
            except (subprocess.TimeoutExpired, OSError, ValueError) as e:
                out[kind] = {"error": f"{type(e).__name__}: {e}"}
                continue
            if kind == "decode":
                mean_ctx = ctx + args.warmup + args.steps / 2
                peak_of = {"products": "GB/s", "head": "GB/s", "attention": "GB/s"}
                extra = {"attention": (args.batch * mean_ctx * nums["kv_bytes_per_token"], 0)}
                out[kind] = account(calls, rows, args.steps, peak_of, measured, extra)
                n_steps, title = args.steps, f"decode step, batch {args.batch}, {ctx}-token contexts"
            else:
                T = prefill_tokens
                peak_of = {"products": "TFLOP/s", "attention": "TFLOP/s", "head": "GB/s", "flops_peak": PEAK_FLOPS[args.dtype]}
                extra = {"attention": (0, cfg.num_hidden_layers * 4.0 * cfg.num_attention_heads * cfg.head_dim * (T * (T + 1) / 2))}
                out[kind] = account(calls, rows, 1, peak_of, measured, extra)
                n_steps, title = 1, f"prefill of one {T}-token prompt in one step"
            if args.profile_out and "all" in out[kind]:
                os.makedirs(args.profile_out, exist_ok=True)
                shape = SHAPES[args.shape][0]
                name = (f"decode_b{args.batch}" + (f"_ctx{ctx}" if ctx != 2048 else "") if kind == "decode" else f"prefill_{T}")
                name += ("" if args.shape == "0.5b" else "_" + args.shape) + ("" if args.dtype == "bf16" else "_" + args.dtype)
                command = "python bench.py " + " ".join(a for a in sys.argv[1:])
                write_summary(os.path.join(args.profile_out, name + ".md"), f"{title} ({shape} shape, {args.dtype}, random weights)", command,
                              out[kind], by_name(rows, n_steps * out[kind]["all"]["launches"]), n_steps, out[kind].get("_work_of"))
            if isinstance(out[kind], dict):
                out[kind].pop("_work_of", None)  # for the summaries only: the record keeps to the kinds
    return out


if __name__ == "__main__":
    sys.exit(main())
