"""Command line in the manner of the reference's `dinfer` binary (bins/dinfer/src/main.rs:28-151).

The reference's `serve` starts an HTTP server; servers and tokenizers are outside this
engine, so the command here is `generate`: token ids in, token ids out, with the engine
flags under the reference's names and defaults. `device-info` prints the device.
"""
from __future__ import annotations

import argparse
import json
import sys


def _engine_flags(p: argparse.ArgumentParser) -> None:
    p.add_argument("--model", required=True, help="folder with config.json and safetensors")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--max-model-len", type=int, default=4096, help="most tokens (prompt + output) of a request")
    p.add_argument("--max-num-seqs", type=int, default=16, help="most live requests")
    p.add_argument("--max-num-batched-tokens", type=int, default=2048, help="token budget of a step")
    p.add_argument("--num-blocks", type=int, default=None, help="cache pages; absent: from free memory")
    p.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    p.add_argument("--gpu-memory-utilization", type=float, default=0.9)
    p.add_argument("--no-decode-exempt", action="store_true", help="decode rows count against the token budget")
    p.add_argument("--enable-prefix-caching", dest="prefix_caching", action="store_true",
                   help="keep the pages of finished requests by their tokens; a prompt with the same start reuses them")
    p.add_argument("--no-prefix-caching", dest="prefix_caching", action="store_false",
                   help="do not reuse pages between requests (default: reuse where every layer keeps all its keys)")
    p.set_defaults(prefix_caching=None)
    p.add_argument("--long-prefill-token-threshold", type=int, default=0,
                   help="most prompt tokens of one request per step (0: no limit)")
    p.add_argument("--prefill-tokens-per-step", type=int, default=0,
                   help="most prompt tokens of all requests per step (0: no limit)")
    p.add_argument("--no-hip-graph", "--no-cuda-graph", dest="no_graph", action="store_true",
                   help="run decode steps eagerly instead of replaying captured graphs")
    p.add_argument("--no-async-scheduling", dest="no_async", action="store_true",
                   help="plan each step only after the tokens of the one before have been read")
    p.add_argument("--gemm-tuning", choices=["measured", "heuristic"], default="measured",
                   help="library products: time the library's candidates once per shape at start-up and keep the "
                        "choices in a file (measured), or take its first suggestion (heuristic)")
    p.add_argument("--max-logits-rows", type=int, default=None,
                   help="rows of logits a step can return (default: one per live request); --prompt-logprobs needs "
                        "more than --max-num-seqs")
    p.add_argument("--device", type=int, default=0)


def _options(a):
    from .config import EngineOptions
    return EngineOptions(
        dtype=a.dtype, max_model_len=a.max_model_len, max_num_seqs=a.max_num_seqs,
        max_num_batched_tokens=a.max_num_batched_tokens, num_blocks=a.num_blocks, block_size=a.block_size,
        gpu_memory_utilization=a.gpu_memory_utilization, decode_exempt_from_budget=not a.no_decode_exempt,
        enable_prefix_caching=a.prefix_caching,
        long_prefill_token_threshold=a.long_prefill_token_threshold,
        prefill_tokens_per_step=a.prefill_tokens_per_step, hip_graph=not a.no_graph, async_scheduling=not a.no_async,
        device=a.device, max_logits_rows=a.max_logits_rows,
        gemm_tuning=a.gemm_tuning)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="dinfer", description="MI355X-native inference engine (token ids in and out)")
    sub = ap.add_subparsers(dest="cmd", required=True)

    g = sub.add_parser("generate", help="generate token ids for prompts given as token ids")
    _engine_flags(g)
    g.add_argument("--prompt-ids", action="append", default=[], help="a prompt as comma-separated token ids (repeatable)")
    g.add_argument("--prompts-file", help="JSON lines, each a list of token ids or {\"prompt_ids\": [...]}")
    g.add_argument("--max-tokens", type=int, default=256)
    g.add_argument("--min-tokens", type=int, default=0)
    g.add_argument("--temperature", type=float, default=1.0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--top-k", type=int, default=-1)
    g.add_argument("--min-p", type=float, default=0.0)
    g.add_argument("--repetition-penalty", type=float, default=1.0)
    g.add_argument("--frequency-penalty", type=float, default=0.0)
    g.add_argument("--presence-penalty", type=float, default=0.0)
    g.add_argument("--seed", type=int, default=None)
    g.add_argument("--stop-token-ids", default="", help="comma-separated extra stop ids")
    g.add_argument("--ignore-eos", action="store_true")
    g.add_argument("--logprobs", type=int, default=None,
                   help="with every output token: its log-probability, rank and this many most probable tokens")
    g.add_argument("--prompt-logprobs", type=int, default=None, help="the same for every prompt token but the first")
    g.add_argument("--logit-bias", default="", help="token:bias pairs, comma-separated, added to those logits")

    r = sub.add_parser("random-weights", help="write a model folder with random weights from a config.json")
    r.add_argument("--config", required=True, help="a config.json of a registered architecture")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])

    d = sub.add_parser("device-info", help="print the device's name and properties")
    d.add_argument("--ordinal", type=int, default=0)

    a = ap.parse_args(argv)
    if a.cmd == "device-info":
        import torch
        if not torch.cuda.is_available():
            print("no HIP device is visible", file=sys.stderr)
            return 1
        p = torch.cuda.get_device_properties(a.ordinal)
        print(json.dumps({"ordinal": a.ordinal, "name": p.name, "arch": getattr(p, "gcnArchName", ""),
                          "compute_units": p.multi_processor_count, "memory_gib": round(p.total_memory / 2**30, 1)}))
        return 0
    if a.cmd == "random-weights":
        from .config.registry import architecture_of
        from .weights import write_random_model
        cfg_d = json.load(open(a.config))
        cfg = architecture_of(cfg_d).config_class.from_dict(cfg_d)
        print(write_random_model(cfg, a.out, seed=a.seed, dtype=a.dtype))
        return 0

    from . import Engine, SamplingParams
    prompts = [[int(t) for t in s.split(",") if t.strip()] for s in a.prompt_ids]
    if a.prompts_file:
        for line in open(a.prompts_file):
            if line.strip():
                rec = json.loads(line)
                prompts.append(rec["prompt_ids"] if isinstance(rec, dict) else rec)
    if not prompts:
        ap.error("give --prompt-ids or --prompts-file")
    sp = SamplingParams(max_tokens=a.max_tokens, min_tokens=a.min_tokens, temperature=a.temperature, top_p=a.top_p,
                        top_k=a.top_k, min_p=a.min_p, repetition_penalty=a.repetition_penalty,
                        frequency_penalty=a.frequency_penalty, presence_penalty=a.presence_penalty, seed=a.seed,
                        stop_token_ids=[int(t) for t in a.stop_token_ids.split(",") if t.strip()],
                        ignore_eos=a.ignore_eos, logprobs=a.logprobs, prompt_logprobs=a.prompt_logprobs,
                        logit_bias=[(int(t), float(b)) for t, b in (x.split(":") for x in a.logit_bias.split(",") if x.strip())])
    if a.prompt_logprobs is not None and a.max_logits_rows is None:
        a.max_logits_rows = a.max_num_seqs + 256
    eng = Engine(a.model, options=_options(a))
    shown = lambda x: None if x is None else {"token_id": x.token_id, "logprob": x.logprob, "rank": x.rank, "top": x.top}
    for p, g in zip(prompts, eng.generate(prompts, sp, details=True)):
        rec = {"prompt_ids": p, "output_ids": g.token_ids, "finish_reason": g.finish_reason}
        if g.logprobs is not None:
            rec["logprobs"] = [shown(x) for x in g.logprobs]
        if g.prompt_logprobs is not None:
            rec["prompt_logprobs"] = [shown(x) for x in g.prompt_logprobs]
        print(json.dumps(rec))
    return 0


if __name__ == "__main__":
    sys.exit(main())
