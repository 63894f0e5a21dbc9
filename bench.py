#!/usr/bin/env python3
"""In-process throughput of the engine on one MI355X: Qwen3-8B-shaped random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L] [--shape 8b|14b|32b|0.6b]
                    [--prompt P] [--context C] [--workload decode|serving [--sampled]]
    python bench.py --workload closed --shape 0.6b --concurrency 8 --prompt 128 --max-tokens 128 [--num-requests N]

Prints ONE JSON line. `value` is decoded tokens per second at the default batch (8), each
request with a 2,048-token prompt in a 4,096-token context; a "step" is one decode step
through the engine's entry point (schedule, batch build, model step, greedy sampling,
token ids back on the host). On the same line:

  prefill   tokens per second of one 2,048-token prompt step; `frac` = the step's flops /
            time / the dense bf16 MFMA peak (2.5 PFLOP/s; fp32: 157.3 TFLOP/s);
  roofline  the decode step against HBM: bytes it has to read (every weight it uses once,
            and the cache of the live requests) / time, against 8 TB/s;
  points    decode tokens per second at batch 1 and 64;
  and, beside the vendor's figures, what this chip delivers to a kernel that does nothing else, measured before
  the timed region: `peak_measured` in roofline (a kernel that only reads 4 GB) and in prefill (chains of bf16
  MFMAs on registers), with `frac_measured` against them;
  phases    where a decode step's time goes (ms a step, from a second, instrumented run of the same steps that
            is not the one timed): the host's schedule, fill, launch, sample, wait and update, and the model's
            kernels on the device between two events (`gpu`);
  gemm      which of the library's algorithms the products of many rows run with (index in its list per shape),
            and how each was chosen.

All data is synthetic: weights N(0, 0.02) / gains 1 + N(0, 0.1) drawn on the device, token
ids uniform in the vocabulary. The reference publishes no number for this size or
hardware, so vs_baseline is null.
"""
import argparse
import json
import random
import sys
import time
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))

# Qwen3-8B layer sizes: the default run
SIZES = dict(vocab_size=151936, hidden_size=4096, intermediate_size=12288, num_hidden_layers=36,
             num_attention_heads=32, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6,
             max_position_embeddings=40960, tie_word_embeddings=False)
# further sizes of the same architecture (Qwen3-14B and 32B); `--shape` picks one
SHAPES = {
    "8b": {},
    "14b": dict(hidden_size=5120, intermediate_size=17408, num_hidden_layers=40, num_attention_heads=40),
    "32b": dict(hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64),
    # the size the reference publishes its own numbers for (models/qwen3/src/config.rs:84-101)
    "0.6b": dict(hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16,
                 tie_word_embeddings=True),
}
DEFAULT_PROMPT, DEFAULT_CONTEXT = 2048, 4096
HBM_PEAK = 8.0e12
MFMA_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}


def model_numbers(c, dtype_bytes):
    Hd, I, L = c["hidden_size"], c["intermediate_size"], c["num_hidden_layers"]
    H, Hkv, D, V = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"], c["vocab_size"]
    per_layer = (H + 2 * Hkv) * D * Hd + H * D * Hd + 3 * I * Hd
    gains = L * (2 * Hd + 2 * D) + Hd
    return dict(linear_params=L * per_layer, head_params=V * Hd, gains=gains,
                kv_bytes_per_token=L * 2 * Hkv * D * dtype_bytes)


def gemm_summary(chosen):
    """The library's algorithm per product shape, short: 'rows x n x k[+]' -> index in its list ('+': adds into its output)."""
    measured = sum(1 for c in chosen if c["chosen"] == "measured")
    picks = {f"{c['m']}x{c['n']}x{c['k']}{'+' if c['accumulate'] else ''}": c["algorithm"]
             for c in chosen if c["m"] in (64, 2048)}
    return {"shapes": len(chosen), "measured": measured, "algorithm_of": picks}


def serving(a, torch, Engine, SamplingParams, Qwen3Config) -> int:
    """32 requests arrive at once: prompts uniform in [512, 3072] tokens, a step budget of 512 prompt tokens beside
    the decoding requests, 256 outputs each. The workload runs `--runs` times (2) on one engine, with new tokens
    each time; the last run is the one reported (the first, also given, pays for first uses: kernel loads, measuring product shapes, graph capture)."""
    sizes = {**SIZES, **SHAPES[a.shape]}
    if a.layers:
        sizes["num_hidden_layers"] = a.layers
    cfg = Qwen3Config.from_dict(sizes)
    n_req, out_len, budget, ctx = 32, 256, 512, 4096
    eng = Engine(config=cfg, seed=0, dtype=a.dtype, max_model_len=ctx, max_num_seqs=n_req, max_num_batched_tokens=budget,
                 block_size=16, num_blocks=n_req * ctx // 16 + 64, hip_graph=not a.no_hip_graph)
    rng = random.Random(0)
    lengths = [rng.randint(512, 3072) for _ in range(n_req)]
    sp = (SamplingParams(max_tokens=out_len, temperature=0.7, top_k=50, top_p=0.9, presence_penalty=0.5, seed=3, ignore_eos=True)
          if a.sampled else SamplingParams(max_tokens=out_len, temperature=0.0, ignore_eos=True))
    def run(phases=False):
        for n in lengths:   # new tokens every run: the prefix cache has nothing to offer
            eng.add_request([rng.randrange(cfg.vocab_size) for _ in range(n)], sp)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = mixed = outs = 0
        t_mixed = 0.0
        split = {"with_prompt_portions": {}, "decode_only": {}}
        while eng.has_unfinished():
            if phases:
                eng.measure_phases(True)
            ts = time.perf_counter()
            got = eng.step()
            steps += 1
            outs += sum(1 for o in got if o.token is not None)
            is_mixed = eng.runner.batch.num_tokens != eng.runner.batch.num_reqs
            if is_mixed:
                mixed += 1
                t_mixed += time.perf_counter() - ts
            if phases:
                acc = split["with_prompt_portions" if is_mixed else "decode_only"]
                for k, v in eng.phases.items():
                    acc[k] = acc.get(k, 0.0) + v
        torch.cuda.synchronize()
        if phases:
            eng.measure_phases(False)
            for acc in split.values():
                n = max(acc.pop("steps", 0), 1)
                for k in acc:
                    acc[k] = round(acc[k] / n * 1e3, 3)
        return time.perf_counter() - t0, steps, mixed, outs, t_mixed, split

    # the first run pays for first uses: kernels load, graphs are captured
    results = [run() for _ in range(max(1, a.runs))]
    cold = results[0][0]
    dt, steps, mixed, outs, t_mixed, _ = results[-1]
    phase_ms = run(phases=True)[5]   # once more with the host's clock around every phase (ms a step); not the timed run
    ptoks = sum(lengths)
    print(json.dumps({
        "metric": f"tokens/s, prompt and output (Qwen3-{a.shape.upper()} shape, 32 requests, prompts 512-3072 in portions of 512, 256 outputs each)",
        "value": round((ptoks + outs) / dt, 1), "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
        "vs_baseline": None, "dtype": "bf16" if a.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "seconds": round(dt, 3), "runs": len(results), "seconds_first_run": round(cold, 3), "prompt_tokens": ptoks, "output_tokens": outs, "output_tokens_per_s": round(outs / dt, 1),
        "steps": steps, "steps_with_prompt_portions": mixed, "seconds_in_those": round(t_mixed, 3), "phases_ms": phase_ms,
        "sampling": "temperature 0.7, top-k 50, top-p 0.9, presence penalty 0.5" if a.sampled else "greedy",
        "config": {"model": f"Qwen3-{a.shape.upper()} shape, random weights", "layers": sizes["num_hidden_layers"],
                   "requests": n_req, "token_budget": budget, "context": ctx, "parallelism": "single GPU"}}))
    return 0


def closed(a, torch, Engine, SamplingParams, Qwen3Config) -> int:
    """The load of the reference's own serving bench without the server (bins/bench/src/main.rs:1-16,
    scripts/verify/bench_compare.sh:36-66): `concurrency` requests are live at any time, each with a fresh prompt of
    `prompt` random tokens and `max_tokens` greedy outputs (eos ignored); when one ends the next is added, until
    `num_requests` (default: four per worker, at least 16) are done. The first two requests of every worker's
    worth are not special here: the whole workload runs once untimed first (kernel loads, product shapes, graphs).
    TTFT = first token on the host - arrival; TPOT = (latency - TTFT) / (outputs - 1)."""
    sizes = {**SIZES, **SHAPES[a.shape]}
    if a.layers:
        sizes["num_hidden_layers"] = a.layers
    cfg = Qwen3Config.from_dict(sizes)
    c, P, O = a.concurrency, a.prompt, a.max_tokens
    n_req = a.num_requests or max(16, 4 * c)
    ctx = -(-(P + O + 1) // 16) * 16
    eng = Engine(config=cfg, seed=0, dtype=a.dtype, max_model_len=ctx, max_num_seqs=c, max_num_batched_tokens=max(2048, P),
                 block_size=16, num_blocks=c * ctx // 16 + 64, hip_graph=not a.no_hip_graph)
    rng = random.Random(0)
    sp = SamplingParams(max_tokens=O, temperature=0.0, ignore_eos=True)

    def run():
        arrived, first, ended, outs = {}, {}, {}, {}
        added = 0
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while added < n_req or eng.has_unfinished():
            while added < n_req and len(arrived) - len(ended) < c:
                rid = eng.add_request([rng.randrange(cfg.vocab_size) for _ in range(P)], sp)
                arrived[rid], outs[rid] = time.perf_counter(), 0
                added += 1
            got = eng.step()
            now = time.perf_counter()
            for o in got:
                if o.token is not None:
                    outs[o.request_id] += 1
                    first.setdefault(o.request_id, now)
                if o.finished:
                    ended[o.request_id] = now
        dt = time.perf_counter() - t0
        ttft = sorted((first[r] - arrived[r]) * 1e3 for r in arrived)
        tpot = sorted((ended[r] - first[r]) / (outs[r] - 1) * 1e3 for r in arrived if outs[r] > 1)
        lat = sorted((ended[r] - arrived[r]) * 1e3 for r in arrived)
        return dt, sum(outs.values()), ttft, tpot, lat

    run()
    dt, n_out, ttft, tpot, lat = run()
    pct = lambda xs, q: round(xs[min(len(xs) - 1, int(q * len(xs)))], 3) if xs else None
    print(json.dumps({
        "metric": f"output tokens/s, closed loop (Qwen3-{a.shape.upper()} shape, {c} live requests, prompts of {P}, {O} outputs each)",
        "value": round(n_out / dt, 1), "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "vs_baseline": None,
        "dtype": "bf16" if a.dtype == "bfloat16" else "fp32", "data": "synthetic", "seconds": round(dt, 3),
        "requests": n_req, "requests_per_s": round(n_req / dt, 2), "output_tokens": n_out,
        "total_tokens_per_s": round((n_out + n_req * P) / dt, 1),
        "ttft_ms": {"p50": pct(ttft, 0.5), "p99": pct(ttft, 0.99)}, "tpot_ms": {"p50": pct(tpot, 0.5), "p99": pct(tpot, 0.99)},
        "latency_ms": {"p50": pct(lat, 0.5)}, "counters": eng.stats(),
        "config": {"model": f"Qwen3-{a.shape.upper()} shape, random weights", "layers": sizes["num_hidden_layers"],
                   "concurrency": c, "prompt_len": P, "max_tokens": O, "context": ctx, "parallelism": "single GPU",
                   "in_process": True}}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (named in config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--no-hip-graph", action="store_true")
    ap.add_argument("--skip-prefill", action="store_true", help="do not time the 2,048-token prefill (profiling decode)")
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="layer sizes (default: Qwen3-8B)")
    ap.add_argument("--prompt", type=int, default=DEFAULT_PROMPT, help="prompt tokens per request (and of the timed prefill)")
    ap.add_argument("--context", type=int, default=DEFAULT_CONTEXT, help="max_model_len the engine is built for")
    ap.add_argument("--workload", default="decode", choices=["decode", "serving", "closed"],
                    help="serving: 32 requests with prompts of 512 to 3,072 tokens fed in portions of 512 beside the "
                         "requests that decode, 256 outputs each (meant for the 14B shape); closed: --concurrency "
                         "requests live at any time, --prompt tokens in and --max-tokens out each, the load of the "
                         "reference's own serving bench without the server; each its own JSON line")
    ap.add_argument("--concurrency", type=int, default=8, help="closed: live requests")
    ap.add_argument("--max-tokens", type=int, default=128, help="closed: outputs per request")
    ap.add_argument("--num-requests", type=int, default=0, help="closed: requests in all (0: four per live request, at least 16)")
    ap.add_argument("--runs", type=int, default=2,
                    help="serving: the workload runs this many times on one engine and the last run is reported")
    ap.add_argument("--sampled", action="store_true",
                    help="serving: temperature 0.7, top-k 50, top-p 0.9 and a presence penalty instead of greedy")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py measures one GPU only (this engine does not use a second one); got --gpus {a.gpus}")
        return 2

    import torch
    from dinfer_amd import Engine, SamplingParams
    from dinfer_amd.config.qwen3 import Qwen3Config
    if a.workload == "serving":
        return serving(a, torch, Engine, SamplingParams, Qwen3Config)
    if a.workload == "closed":
        return closed(a, torch, Engine, SamplingParams, Qwen3Config)

    sizes = {**SIZES, **SHAPES[a.shape]}
    PROMPT, CONTEXT = a.prompt, a.context
    if not 0 < PROMPT < CONTEXT:
        print("--prompt must lie below --context")
        return 2
    full_layers = sizes["num_hidden_layers"]
    if a.layers:
        sizes["num_hidden_layers"] = a.layers
    cfg = Qwen3Config.from_dict(sizes)
    dbytes = 2 if a.dtype == "bfloat16" else 4
    nums = model_numbers(sizes, dbytes)
    max_b = max(a.batch, 1 if a.no_points else 64)
    page = 16
    # the cache of max_b requests of the whole context must fit beside the weights: at long contexts the
    # largest point is left out rather than the run refused
    total_mem = torch.cuda.get_device_properties(0).total_memory
    weight_mem = (nums["linear_params"] + 2 * nums["head_params"]) * dbytes
    fits = int((0.85 * total_mem - weight_mem) // (CONTEXT * nums["kv_bytes_per_token"]))
    if fits < a.batch:
        print(f"the cache of {a.batch} requests of {CONTEXT} tokens does not fit this GPU beside the weights ({fits} do)")
        return 2
    max_b = min(max_b, fits)
    eng = Engine(config=cfg, seed=0, dtype=a.dtype, max_model_len=CONTEXT, max_num_seqs=max_b,
                 max_num_batched_tokens=PROMPT, block_size=page, num_blocks=max_b * CONTEXT // page + 64,
                 hip_graph=not a.no_hip_graph)
    rng = random.Random(0)
    V = cfg.vocab_size
    # what the chip gives a kernel that only reads, and one that only multiplies (before anything is timed)
    from dinfer_amd.kernels import blaslt, ops
    hbm_measured = ops.measured_hbm_read(eng.runner.device)
    mfma_measured = ops.measured_mfma_bf16(eng.runner.device) if a.dtype == "bfloat16" else None

    def prompt():
        return [rng.randrange(V) for _ in range(PROMPT)]

    def sync():
        torch.cuda.synchronize()

    greedy = SamplingParams(max_tokens=CONTEXT - PROMPT, temperature=0.0, ignore_eos=True)

    # ---- prefill: one request, one step of 2,048 tokens (the step also samples its first token)
    def time_prefill():
        rid = eng.add_request(prompt(), greedy)
        sync()
        t0 = time.perf_counter()
        eng.step()
        sync()
        dt = time.perf_counter() - t0
        eng.abort(rid)
        return dt

    prefill = None
    if not a.skip_prefill:
        time_prefill()  # warm-up: library initialisation, first-use allocations
        pre = min(time_prefill() for _ in range(3))
        attn_flops = sizes["num_hidden_layers"] * 2 * PROMPT * PROMPT * cfg.head_dim * cfg.num_attention_heads
        pre_flops = 2 * PROMPT * nums["linear_params"] + attn_flops + 2 * nums["head_params"]
        prefill = {"value": round(PROMPT / pre, 1), "tokens": PROMPT, "ms": round(pre * 1e3, 3),
                   "frac": round(pre_flops / pre / MFMA_PEAK[a.dtype], 4), "peak": MFMA_PEAK[a.dtype] / 1e12, "unit": "TFLOP/s"}
        if mfma_measured:
            prefill["peak_measured"] = round(mfma_measured / 1e12, 1)
            prefill["frac_measured"] = round(pre_flops / pre / mfma_measured, 4)

    # ---- decode at a batch: B requests prefilled to 2,048 tokens, then timed decode steps
    def decode(batch, steps, warmup, phases=False):
        ids = [eng.add_request(prompt(), greedy) for _ in range(batch)]
        while any(r.num_computed < PROMPT for r in eng.scheduler.requests.values()):
            eng.step()
        for _ in range(warmup):
            eng.step()
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            eng.step()
        sync()
        dt = (time.perf_counter() - t0) / steps
        ctx = PROMPT + 1 + warmup + steps / 2  # mean cached tokens per request over the timed steps
        ph = None
        if phases:      # the same steps once more with the host's clock around every phase; not the timed run
            eng.measure_phases(True)
            for _ in range(steps):
                eng.step()
            sync()
            n = max(eng.phases.pop("steps"), 1)
            ph = {k: round(v / n * 1e3, 4) for k, v in eng.phases.items()}
            eng.measure_phases(False)
        for i in ids:
            eng.abort(i)
        return dt, ctx, ph

    dt, ctx, phases = decode(a.batch, a.steps, a.warmup, phases=True)
    weight_bytes = (nums["linear_params"] + nums["head_params"] + nums["gains"] + a.batch * cfg.hidden_size) * dbytes
    step_bytes = weight_bytes + a.batch * ctx * nums["kv_bytes_per_token"]
    achieved = step_bytes / dt
    points = {}
    if not a.no_points:
        for b in (1, 64):
            if b > max_b:
                continue
            d, _, _ = decode(b, a.steps, a.warmup)
            points[f"decode_b{b}"] = round(b / d, 1)

    line = {
        "metric": f"decode tok/s (Qwen3-{a.shape.upper()} shape, batch {a.batch}, {PROMPT}-token prompts, context {CONTEXT})",
        "value": round(a.batch / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if a.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": f"Qwen3-{a.shape.upper()} shape, random weights", "global_batch": a.batch, "seq_len": CONTEXT,
            "prompt_len": PROMPT, "parallelism": "single GPU", "layers": sizes["num_hidden_layers"],
            "layers_of_config": full_layers, "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size,
            "vocab": cfg.vocab_size, "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps,
            "tied_head": cfg.tie_word_embeddings, "page_size": page, "hip_graph": not a.no_hip_graph,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4), "peak_measured": round(hbm_measured / 1e9, 1),
                     "frac_measured": round(achieved / hbm_measured, 4)},
        "points": points,
        "phases": phases,
        "gemm": gemm_summary(blaslt.chosen()),
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
