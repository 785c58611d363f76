"""Headline benchmark: decode tokens/s (batch 8 by default) and prefill tokens/s at 2,048
tokens for GPT-2 small sizes with random weights on one MI355X, with roofline fractions.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--dtype bfloat16]

A "step" is one decode step of the whole engine (scheduler, step function, kernels,
sampling). Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12                                   # bytes/s
MFMA_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}


SIZES = {   # the benchmark configurations' sizes (GPT-2 small, medium, XL): n_layer, n_embd, n_head, n_inner
    "gpt2-small": (12, 768, 12, 3072), "gpt2-medium": (24, 1024, 16, 4096), "gpt2-xl": (48, 1600, 25, 6400),
}


def small_config(n_layer, size="gpt2-small", n_positions=1024):
    full_layers, d, h, f = SIZES[size]
    return dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=n_layer or full_layers, n_embd=d,
                n_head=h, n_inner=f, vocab_size=50257, n_positions=n_positions, layer_norm_epsilon=1e-5,
                activation_function="gelu_new", eos_token_id=50256, bos_token_id=50256)


def decode_run(model_dir, dtype, batch, prompt_len, steps, warmup, cfg):
    """Decode steps of `batch` requests through the whole engine. Every prompt is fed in ONE step before
    the clock starts, so that all requests decode in lockstep from position prompt_len on. Returns
    tokens/s, mean and median seconds per step, the mean context length, and the bytes one step has to
    read (every weight once, and the cache of the live requests), taken from the model's parts and the cache."""
    import torch
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    pages = batch * (cfg["n_positions"] // 16) + 16
    options = EngineOptions(kv_block_size=16, total_kv_blocks=pages, max_batch_num=max(batch, 1),
                            max_tokens_per_step=batch * prompt_len, prefill_chunk=prompt_len)
    engine = Engine.from_pretrained(model_dir, dtype=dtype, options=options)
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, cfg["vocab_size"], (prompt_len,), generator=g).tolist() for _ in range(batch)]
    # The workload generates up to 512 tokens per request (as many as the positions allow); the timed
    # steps are taken from the middle of that stretch, so that their mean context is the workload's.
    room = cfg["n_positions"] - prompt_len - 1
    skip = max(0, min(512, room) // 2 - steps // 2 - warmup)
    total_new = 1 + skip + warmup + steps
    assert prompt_len + total_new <= cfg["n_positions"], "the run would pass the last position"
    params = SamplingParams(max_new_tokens=total_new, ignore_eos=True)
    for p in prompts:
        engine.add_request(p, params)
    # untimed: the prompts (one step), then the warm-up steps
    engine.step()
    st = engine.stats()
    assert st["prefill_tokens"] == batch * prompt_len and st["steps"] == 1, "the prompts did not fit one step"
    for _ in range(skip + warmup):
        engine.step()
    engine.synchronize()
    ctx0 = prompt_len + 1 + skip + warmup
    per_step = []
    n_tok = 0
    t0 = t_prev = time.perf_counter()
    for _ in range(steps):
        n_tok += len(engine.step())
        t_now = time.perf_counter()
        per_step.append(t_now - t_prev)
        t_prev = t_now
    engine.synchronize()
    dt = time.perf_counter() - t0
    assert n_tok == batch * steps, (n_tok, batch, steps)
    mean_ctx = ctx0 + (steps - 1) / 2.0
    info = engine.runner.info()
    bytes_step = info["weight_bytes"] + batch * mean_ctx * info["cache_bytes_per_token"]
    per_step.sort()
    p50 = per_step[len(per_step) // 2]
    engine.close()
    return n_tok / dt, dt / steps, p50, mean_ctx, bytes_step


def prefill_run(model_dir, dtype, cfg, n_req=2, n_tok=1024, reps=5):
    """One step of n_req whole prompts of n_tok tokens (logits at the last place of each); the best of
    `reps` runs. Flops from the model's parts: products of every token, attention over the causal triangle,
    the head's rows."""
    import torch
    from mini_llm_amd import Runner, StepEntry
    runner = Runner(model_dir=model_dir, dtype=dtype, page_size=16, n_pages=n_req * n_tok // 16 + 8, max_num_seqs=n_req)
    g = torch.Generator().manual_seed(3)
    toks = [torch.randint(0, cfg["vocab_size"], (n_tok,), generator=g).to(torch.int32).numpy() for _ in range(n_req)]
    times = []
    for rep in range(reps + 2):
        entries = [StepEntry(i, toks[i], [n_tok - 1]) for i in range(n_req)]
        runner.synchronize()
        t0 = time.perf_counter()
        runner.step(entries)             # returns with the logits on the host
        times.append(time.perf_counter() - t0)
        for i in range(n_req):
            runner.end_request(i)
    dt = min(times[2:])
    T = n_req * n_tok
    cost = runner.info()
    flops = (float(T) * cost["flops_per_token"] + n_req * cost["attention_flops_per_key"] * (n_tok * (n_tok + 1) / 2)
             + float(n_req) * cost["flops_per_logits_row"])
    del runner
    return T / dt, dt, flops


def serving_run(model_dir, dtype, cfg, n_req, prompt_lo, prompt_hi, new_tokens, max_batch, chunk, pages, seed,
                preempt_for_decode=True):
    """Continuous batching from a full queue: n_req requests with prompt lengths uniform in
    [prompt_lo, prompt_hi] and new_tokens generated each, prompts fed in portions of `chunk`, at most
    max_batch requests a step, `pages` pages of 16 tokens in the pool. Returns a dictionary of
    totals, times and the scheduler's counters."""
    import torch
    from mini_llm_amd import Engine, EngineOptions, SamplingParams
    options = EngineOptions(kv_block_size=16, total_kv_blocks=pages, max_batch_num=max_batch,
                            max_tokens_per_step=max(2048, max_batch + chunk), prefill_chunk=chunk,
                            preempt_for_decode=preempt_for_decode)
    engine = Engine.from_pretrained(model_dir, dtype=dtype, options=options)
    engine.generate([[0]] * min(max_batch, 8), SamplingParams(max_new_tokens=2, ignore_eos=True))     # loads the kernels
    base = engine.stats()
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(prompt_lo, prompt_hi + 1, (n_req,), generator=g).tolist()
    params = SamplingParams(max_new_tokens=new_tokens, ignore_eos=True)
    for n in lens:
        engine.add_request(torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist(), params)
    engine.synchronize()
    t0 = time.perf_counter()
    n_out = n_steps = failed = 0
    first = None
    first_at, last_at, count = {}, {}, {}          # per request: when its first and its last token arrived, how many
    while engine.has_unfinished():
        outs = engine.step()
        n_steps += 1
        now = time.perf_counter() - t0
        if outs and first is None:
            engine.synchronize()
            first = now = time.perf_counter() - t0
        for o in outs:
            if o.token >= 0:
                n_out += 1
                first_at.setdefault(o.request_id, now)
                last_at[o.request_id] = now
                count[o.request_id] = count.get(o.request_id, 0) + 1
            else:
                failed += 1
    engine.synchronize()
    dt = time.perf_counter() - t0
    # as the host sees them (tokens arrive one step late): time to the first token, time per later token, whole request
    ttft = sorted(first_at.values())
    e2e = sorted(last_at.values())
    tpot = [(last_at[r] - first_at[r]) / (count[r] - 1) for r in count if count[r] > 1]
    pct = lambda v, q: v[min(len(v) - 1, int(q * len(v)))] if v else 0.0
    latency = {"ttft_ms_p50": round(1e3 * pct(ttft, 0.5), 2), "ttft_ms_p99": round(1e3 * pct(ttft, 0.99), 2),
               "tpot_ms_mean": round(1e3 * sum(tpot) / max(len(tpot), 1), 3),
               "e2e_ms_p50": round(1e3 * pct(e2e, 0.5), 1), "e2e_ms_p99": round(1e3 * pct(e2e, 0.99), 1)}
    st = engine.stats()
    for k in ("preemptions", "deferred_decodes", "deferred_prefills"):
        st[k] -= base[k]
    assert n_out == (n_req - failed) * new_tokens, (n_out, n_req, failed, new_tokens)
    assert st["free_pages"] == pages and engine.runner.check() == ""
    return {"seconds": dt, "generated": n_out, "prompt_tokens": sum(lens), "steps": n_steps,
            "first_token_s": first, "failed": failed, "counters": st, "latency": latency}


def serving_main(args, cfg, model_dir):
    """--workload continuous: 64 requests with prompts of 64 to 768 tokens and 256 new tokens each, portions
    of 256 (the workload made for GPT-2 medium sizes); --workload kv-pressure: 256 requests of 512 + 512
    tokens (made for GPT-2 XL sizes), the pool capped at 60 % of what the 64 requests of a full batch hold
    at their end, so that requests are deferred and preempted."""
    if args.workload == "continuous":
        n_req, lo, hi, new, max_batch, chunk = 64, 64, 768, 256, 64, 256
        pages = n_req * ((hi + new + 15) // 16) + 16
    else:
        n_req, lo, hi, new, max_batch, chunk = 256, 512, 512, 512, 64, 512
        pages = int(0.6 * max_batch * ((hi + new + 15) // 16))
    r = serving_run(model_dir, args.dtype, cfg, n_req, lo, hi, new, max_batch, chunk, pages, seed=7,
                    preempt_for_decode=not args.defer_decodes)
    c = r["counters"]
    rec = {"metric": f"generated tok/s, {args.workload} workload ({args.size} sizes)",
           "value": round(r["generated"] / r["seconds"], 1), "unit": "tok/s", "n_gpus": 1,
           "steps": r["steps"], "warmup": 0, "ms_per_step": round(1e3 * r["seconds"] / r["steps"], 4),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
           "data": "synthetic (random weights seed 2, uniform random token ids and prompt lengths, seed 7)"
                   "; a few two-token requests before the clock starts",
           "config": {"model": args.size + "-sizes", "n_layer": cfg["n_layer"], "n_layer_full": SIZES[args.size][0],
                      "requests": n_req, "prompt_min": lo, "prompt_max": hi, "new_tokens": new,
                      "max_batch_num": max_batch, "prefill_chunk": chunk, "kv_blocks": pages, "kv_block_size": 16,
                      "preempt_for_decode": not args.defer_decodes},
           # what the run did (the configuration above holds sizes only)
           "serving": {"prompt_tokens": r["prompt_tokens"], "generated_tokens": r["generated"],
                       "total_tok_per_s": round((r["generated"] + r["prompt_tokens"]) / r["seconds"], 1),
                       "seconds": round(r["seconds"], 3), "first_token_ms": round(1e3 * (r["first_token_s"] or 0), 2),
                       # mean composition of a step: decoded tokens and prompt tokens in it
                       "decode_rows_per_step": round(r["generated"] / r["steps"], 1),
                       "prompt_tokens_per_step": round(r["prompt_tokens"] / r["steps"], 1),
                       "preemptions": c["preemptions"], "deferred_decodes": c["deferred_decodes"],
                       "deferred_prefills": c["deferred_prefills"], "failed": r["failed"], **r["latency"]}}
    print(json.dumps(rec))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the size has (named in config)")
    ap.add_argument("--size", default="gpt2-small", choices=sorted(SIZES), help="layer sizes (default: configs[2])")
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--positions", type=int, default=1024,
                    help="n_positions of the random model (the benchmark's context length; longer: further context lengths)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1/64 and prefill measurements")
    ap.add_argument("--prefill-only", action="store_true", help="measure only the prefill step (profiling)")
    ap.add_argument("--prefill-requests", type=int, default=2, help="with --prefill-only: prompts in the step")
    ap.add_argument("--prefill-tokens", type=int, default=1024, help="with --prefill-only: tokens of each prompt")
    ap.add_argument("--defer-decodes", action="store_true",
                    help="serving workloads: a decode that gets no page waits on its pages (the reference's manner) "
                         "instead of preempting a younger request at once")
    ap.add_argument("--plugin", action="append", default=[],
                    help="a shared library that registers further architectures (with --config)")
    ap.add_argument("--config", help="a config.json to measure in place of the GPT-2 sizes (any registered architecture; "
                                     "it names vocab_size and n_positions, or --vocab / --positions do)")
    ap.add_argument("--vocab", type=int, default=0, help="with --config: the vocabulary to draw token ids from")
    ap.add_argument("--peaks-only", action="store_true",
                    help="measure this GPU's streaming bandwidth and matrix-core rate and print them")
    ap.add_argument("--workload", default="decode", choices=["decode", "continuous", "kv-pressure"],
                    help="decode: the headline measurement; continuous / kv-pressure: a queue of requests "
                         "through the scheduler")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    from mini_llm_amd import load_plugin, write_random_model

    for path in args.plugin:
        load_plugin(path)
    cfg = small_config(args.layers, args.size, args.positions)
    if args.config:
        # another architecture, served by the same engine: sizes from its own config.json
        with open(args.config) as f:
            cfg = json.load(f)
        # (what the measurement itself needs to know: where token ids and positions end; keys the architecture does
        # not read are ignored by it)
        cfg.setdefault("vocab_size", args.vocab or cfg.get("vocab", 0))
        cfg.setdefault("n_positions", args.positions)
        if cfg["vocab_size"] < 1:
            print("bench.py: --config names no vocab_size; give --vocab")
            return 2
        cfg.setdefault("n_layer", None)
        args.size = cfg.get("architectures", ["?"])[0]
        SIZES[args.size] = (cfg["n_layer"], 0, 0, 0)
    if "n_embd" not in cfg:
        args.no_points = True
    if args.peaks_only:
        from mini_llm_amd.kernels.peaks import NOMINAL, measure_peaks
        print(json.dumps({"metric": "measured peaks of this GPU", "measured": measure_peaks("cuda:0"),
                          "published": NOMINAL}))
        return 0
    # all prompts are fed in one step, then 1 + warmup + steps tokens are generated for each request
    room = cfg["n_positions"] - args.prompt_len - 1
    if room < 2:
        print(f"bench.py: prompts of {args.prompt_len} tokens leave no room to decode in {cfg['n_positions']} positions")
        return 2
    warmup = min(args.warmup, max(1, room // 6)) if args.warmup + args.steps > room else args.warmup
    steps = min(args.steps, room - warmup)
    with tempfile.TemporaryDirectory() as d:
        write_random_model(dict(cfg), d, seed=2)
        if args.workload != "decode":
            return serving_main(args, cfg, d)
        if args.prefill_only:
            ptps, pdt, flops = prefill_run(d, args.dtype, cfg, args.prefill_requests, args.prefill_tokens)
            print(json.dumps({"metric": f"prefill tok/s at {args.prefill_requests} x {args.prefill_tokens} tokens "
                                        f"({args.size} sizes)", "value": round(ptps, 1), "unit": "tok/s",
                              "ms": round(pdt * 1e3, 4), "tflops": round(flops / pdt / 1e12, 1),
                              "frac": round(flops / pdt / MFMA_PEAK[args.dtype], 5)}))
            return 0
        tps, step_s, p50_s, mean_ctx, bytes_step = decode_run(d, args.dtype, args.batch, args.prompt_len, steps,
                                                             warmup, cfg)
        # The reference's own decode numbers at this workload (GPT-2 small, 512-token prompts; fp32 on a
        # TITAN V: /root/reference benchmark gpt2_decode_batch_sweep_512.csv:2-5), where it has one.
        reference_tps = {1: 116.9, 2: 223.1, 4: 438.6, 8: 854.4}.get(args.batch) \
            if (args.size == "gpt2-small" and args.prompt_len == 512 and cfg["n_layer"] == SIZES[args.size][0]) else None
        achieved = bytes_step / step_s
        rec = {
            "metric": f"decode tok/s at batch {args.batch} ({args.size} sizes, {args.prompt_len}-token prompts)",
            "value": round(tps, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(step_s * 1e3, 4), "ms_per_step_p50": round(p50_s * 1e3, 4),
            "higher_is_better": True, "scaling": "weak",
            "vs_baseline": round(tps / reference_tps, 2) if reference_tps else None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic (random weights seed 2, uniform random token ids)",
            "config": {"model": args.size + "-sizes", "n_layer": cfg["n_layer"], "n_layer_full": SIZES[args.size][0],
                       "n_embd": cfg.get("n_embd"), "n_head": cfg.get("n_head"),
                       "head_dim": cfg["n_embd"] // cfg["n_head"] if "n_embd" in cfg else None,
                       "n_inner": cfg.get("n_inner"), "vocab_size": cfg["vocab_size"],
                       "n_positions": cfg["n_positions"], "global_batch": args.batch,
                       "prompt_len": args.prompt_len, "seq_len": cfg["n_positions"],
                       "mean_context": round(mean_ctx, 1), "kv_block_size": 16, "parallelism": "single-gpu",
                       "engine": "native (the one behind bin/mini-llm)",
                       "baseline": (f"{reference_tps} tok/s: the reference, fp32, TITAN V" if reference_tps else "none")},
            "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 2), "peak": HBM_PEAK / 1e9,
                         "unit": "GB/s", "frac": round(achieved / HBM_PEAK, 5),
                         "bytes_per_step": int(bytes_step)},
        }
        if not args.no_points:
            ptps, pdt, flops = prefill_run(d, args.dtype, cfg)
            rec["prefill"] = {"value": round(ptps, 1), "tokens": 2048, "ms": round(pdt * 1e3, 4),
                              "frac": round(flops / pdt / MFMA_PEAK[args.dtype], 5)}
            points = {}
            for b in (1, 64):
                s = min(steps, 128)
                v = decode_run(d, args.dtype, b, args.prompt_len, s, min(warmup, 16), cfg)[0]
                points[f"decode_b{b}"] = round(v, 1)
            rec["points"] = points
            # what this GPU gives on the engine's own micro-benchmarks, beside the published peaks
            from mini_llm_amd.kernels.peaks import measure_peaks
            peaks = measure_peaks("cuda:0")
            rec["measured_peaks"] = peaks
            rec["roofline"]["frac_of_measured"] = round(achieved / (peaks["hbm_read_GBps"] * 1e9), 5)
            mfma = peaks["mfma_bf16_TFLOPs" if args.dtype == "bfloat16" else "mfma_f32_TFLOPs"] * 1e12
            rec["prefill"]["frac_of_measured"] = round(flops / pdt / mfma, 5)
    print(json.dumps(rec))
    return 0


if __name__ == "__main__":
    sys.exit(main())
