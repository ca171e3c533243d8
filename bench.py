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


def kugulorn_config(n_layer, size="gpt2-small", n_positions=1024):
    """A Kugulorn model of about the size of the GPT-2 configuration `size`: the same width, number of layers,
    vocabulary and context; Mamba-2 layers (inner width twice the model's, heads of 64, a state of 128 rows) and
    latent-attention layers (as many heads as GPT-2 has, a latent of up to a third of the width beside 32 rotated
    columns, every second one reading the pages of the one before it, the window as long as the context) in
    turn, each with a gated feed-forward whose three matrices hold what GPT-2's two do."""
    full_layers, d, h, f = SIZES[size]
    n = n_layer or full_layers
    rank = max(r for r in (64, 128, 256, 512) if r <= max(64, d // 3))      # 256 at 768 and 1,024, 512 at 1,600
    ff = f * 2 // 3 // 64 * 64
    mlp = {"kind": "dense", "ff": ff, "limit": 7.0}
    layers, last_own = [], None
    for i in range(n):
        if i % 2 == 0:
            layers.append({"type": "mamba2", "mlp": mlp,
                           "mixer": {"heads": 2 * d // 64, "vdim": 64, "state": 128, "groups": 1, "conv": 4, "norm_groups": 1}})
        else:
            m = {"heads": h, "dim": 64, "rot_dim": 32, "vdim": 64, "kv_rank": rank, "q_rank": d // 2, "scale": 96 ** -0.5,
                 "mask": {"size": n_positions}, "rot": {"base": 10000.0, "dims": 32}}
            if last_own is not None and (i // 2) % 2 == 1:
                m["kv_from"] = last_own
            else:
                last_own = i
            layers.append({"type": "latent_attention", "mixer": m, "mlp": mlp})
    return {"architecture": "Kugulorn", "vocab": 50257, "width": d, "residual_mult": 1.0, "norm": {"eps": 1e-6}, "layers": layers,
            # (what the measurement itself reads; the architecture ignores them)
            "vocab_size": 50257, "n_positions": n_positions, "n_layer": n}


def rekirax_config(n_layer, size="gpt2-small", n_positions=1024):
    """A Rekirax model that runs as many layers as the GPT-2 configuration `size` has, at the same width, vocabulary
    and context: layers of chunked attention beside an HGRN2 recurrence (twice) and of windowed attention (once) in
    turn, heads of 64 as many as GPT-2 has, a quarter as many key/value heads, windows and chunks of 512, 32 rotated
    columns, four taps, each layer with a gated feed-forward whose three matrices hold what GPT-2's two do; the
    layers 1 to 3 run twice (so the list is three layers shorter than the number of runs)."""
    full_layers, d, h, f = SIZES[size]
    runs = n_layer or full_layers
    n = max(runs - 3, 4)
    kv = max(k for k in range(1, max(h // 4, 1) + 1) if h % k == 0)
    mlp = {"kind": "dense", "ff": f * 2 // 3 // 64 * 64}
    layers = []
    for i in range(n):
        if i % 3 == 2:
            layers.append({"type": "attention", "mlp": mlp,
                           "mixer": {"heads": h, "kv_heads": kv, "dim": 64, "vdim": 64, "scale": 0.125, "softcap": 30.0, "mask": {"size": 512}}})
        else:
            left = {"heads": h, "kv_heads": kv, "dim": 64, "vdim": 64, "scale": 0.125, "mask": {"size": 512}, "rot": {"base": 10000.0, "dims": 32}}
            layers.append({"type": "parallel", "mlp": mlp, "mixer": {"left": left, "right": {"heads": h, "dim": 64, "vdim": 64}}})
    return {"architecture": "Rekirax", "vocab": 50257, "width": d, "norm": {"eps": 1e-6}, "canon": {"taps": 4},
            "loop": {"start": 1, "stop": 4, "times": 2}, "layers": layers,
            # (what the measurement itself reads; the architecture ignores them)
            "vocab_size": 50257, "n_positions": n_positions, "n_layer": n + 3}


def viladra_config(n_layer, size="gpt2-small", n_positions=1024):
    """A Viladra model with as many layers as the GPT-2 configuration `size` has, at the same width, vocabulary and
    context: linear attention with a decay per key channel (gla), retention and windowed sigmoid attention in turn,
    heads of 64 as many as GPT-2 has (a quarter as many key/value heads, a window of 512, 32 rotated columns, decays'
    maps of rank 16), four taps, each layer with eight experts of which two are chosen beside a shared one; all
    experts together hold what GPT-2's two feed-forward matrices do (the shared one a quarter of it)."""
    full_layers, d, h, f = SIZES[size]
    n = n_layer or full_layers
    kv = max(k for k in range(1, max(h // 4, 1) + 1) if h % k == 0)
    mlp = {"kind": "moe", "router": {"experts": 8, "top": 2, "scale": 2.0}, "expert": {"ff": 3 * f // 32}, "shared": {"ff": f // 4}}
    layers = []
    for i in range(n):
        if i % 3 == 0:
            layers.append({"type": "gla", "mlp": mlp, "mixer": {"heads": h, "dim": 64, "vdim": 64, "tau": 16.0, "rank": 16}})
        elif i % 3 == 1:
            layers.append({"type": "retention", "mlp": mlp,
                           "mixer": {"heads": h, "dim": 64, "vdim": 64, "decay": [1.0 - 2.0 ** -(5 + 5 * k / h) for k in range(h)],
                                     "rot": {"base": 10000.0, "dims": 32}}})
        else:
            layers.append({"type": "attention", "mlp": mlp,
                           "mixer": {"heads": h, "kv_heads": kv, "dim": 64, "vdim": 64, "scale": 0.125, "mask": {"size": 512}}})
    return {"architecture": "Viladra", "vocab": 50257, "width": d, "norm": {"eps": 1e-6}, "canon": {"taps": 4},
            "embedding": {"scale": 1.0}, "logit_softcap": 30.0, "layers": layers,
            # (what the measurement itself reads; the architecture ignores them)
            "vocab_size": 50257, "n_positions": n_positions, "n_layer": n}


def sunulorn_config(n_layer, size="gpt2-small", n_positions=1024):
    """A Sunulorn model with as many layers as the GPT-2 configuration `size` has, at the same width, vocabulary and
    context: its three attentions in turn (a convolution of four taps over queries and keys with 32 interleaved rotated
    columns; a window of 512 that keeps the first 16 positions, all 64 columns rotated; a distance penalty, a sink and
    a gate per head, every second such layer reading the keys and values of the one before it), heads of 64 as many as
    GPT-2 has and a quarter as many key/value heads; a gated feed-forward and eight clamped gated experts of which two
    are chosen beside a shared one in turn, each holding what GPT-2's two feed-forward matrices do."""
    full_layers, d, h, f = SIZES[size]
    n = n_layer or full_layers
    kv = max(k for k in range(1, max(h // 4, 1) + 1) if h % k == 0)
    dense = {"kind": "dense", "ff": f * 2 // 3 // 64 * 64}
    moe = {"kind": "moe", "router": {"experts": 8, "top": 2}, "expert": {"ff": f // 16, "limit": 7.0}, "shared": {"ff": f // 6 // 64 * 64, "limit": 7.0}}
    layers, last_own = [], None
    for i in range(n):
        mlp = dense if i % 2 == 0 else moe
        base = {"heads": h, "kv_heads": kv, "dim": 64, "vdim": 64, "scale": 0.125}
        if i % 3 == 0:
            layers.append({"type": "attention", "mlp": mlp, "mixer": dict(base, conv=4, rot={"base": 10000.0, "dims": 32})})
        elif i % 3 == 1:
            layers.append({"type": "attention_2", "mlp": mlp,
                           "mixer": dict(base, rot={"base": 10000.0, "dims": 64}, mask={"size": 512, "keep_first": 16})})
        else:
            m = dict(base)
            if last_own is not None and (i // 3) % 2 == 1:
                m["kv_from"] = last_own
            else:
                last_own = i
            layers.append({"type": "attention_3", "mlp": mlp, "mixer": m})
    return {"architecture": "Sunulorn", "vocab": 50257, "width": d, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0}, "layers": layers,
            # (what the measurement itself reads; the architecture ignores them)
            "vocab_size": 50257, "n_positions": n_positions, "n_layer": n}


DESIGNS = {"kugulorn": kugulorn_config, "rekirax": rekirax_config, "viladra": viladra_config, "sunulorn": sunulorn_config}


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
    # (a request's recurrent state, where the model has one, is read and written once a step)
    bytes_step = info["weight_bytes"] + batch * (mean_ctx * info["cache_bytes_per_token"] + 2 * info.get("state_bytes_per_request", 0))
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


def compare_main(args):
    """--compare: both designs at one size through prefill_run and decode_run."""
    from mini_llm_amd import Runner, write_random_model
    other = args.design if args.design in DESIGNS else "kugulorn"
    base = args.beside
    names = {"gpt2": "GPT-2"}
    out = {"metric": f"{other.capitalize()} beside {names.get(base, base.capitalize())} at {args.size} sizes: prefill tok/s (2 x 1,024 tokens) and decode tok/s",
           "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights seed 2, uniform random token ids)",
           "n_gpus": 1, "designs": {}}
    for design in (base, other):
        cfg = (DESIGNS[design] if design in DESIGNS else small_config)(args.layers, args.size, args.positions)
        with tempfile.TemporaryDirectory() as d:
            write_random_model(dict(cfg), d, seed=2)
            r = Runner(model_dir=d, dtype=args.dtype, page_size=16, n_pages=8, max_num_seqs=1)
            info = r.info()
            del r
            ptps, pdt, flops = prefill_run(d, args.dtype, cfg)
            rec = {"n_layer": cfg["n_layer"], "weight_bytes": int(info["weight_bytes"]), "cache_bytes_per_token": info["cache_bytes_per_token"],
                   "state_bytes_per_request": info.get("state_bytes_per_request", 0),
                   "prefill": {"tok_per_s": round(ptps, 1), "ms": round(pdt * 1e3, 4), "tflops": round(flops / pdt / 1e12, 1),
                               "frac_of_peak": round(flops / pdt / MFMA_PEAK[args.dtype], 5)}}
            for b in (1, 8, 64):
                tps, step_s, p50, mean_ctx, bytes_step = decode_run(d, args.dtype, b, args.prompt_len, min(args.steps, 128), min(args.warmup, 16), cfg)
                rec[f"decode_b{b}"] = {"tok_per_s": round(tps, 1), "ms_per_step": round(step_s * 1e3, 4), "mean_context": round(mean_ctx, 1),
                                       "GBps": round(bytes_step / step_s / 1e9, 1), "frac_of_hbm_peak": round(bytes_step / step_s / HBM_PEAK, 5)}
            out["designs"][design] = rec
    g, k = out["designs"][base], out["designs"][other]
    out[other + "_over_" + base] = {"prefill": round(k["prefill"]["tok_per_s"] / g["prefill"]["tok_per_s"], 3),
                                 **{f"decode_b{b}": round(k[f"decode_b{b}"]["tok_per_s"] / g[f"decode_b{b}"]["tok_per_s"], 3) for b in (1, 8, 64)}}
    print(json.dumps(out))
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
    ap.add_argument("--design", default="gpt2", choices=["gpt2", "kugulorn", "rekirax", "viladra", "sunulorn"],
                    help="kugulorn / rekirax / viladra / sunulorn: a model of that design of about the size --size names (kugulorn_config, "
                         "rekirax_config, viladra_config, sunulorn_config) through the same measurement; --compare runs it and GPT-2 one after the other")
    ap.add_argument("--beside", default="gpt2", choices=["gpt2", "kugulorn", "rekirax", "viladra", "sunulorn"],
                    help="with --compare: the design that the --design model is measured beside (default GPT-2)")
    ap.add_argument("--compare", action="store_true",
                    help="prefill (2 x 1,024 tokens) and decode (batch 1, 8, 64) of the --design model (default Kugulorn) and of the GPT-2 model "
                         "of --size, side by side in one JSON line")
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
    if args.compare:
        return compare_main(args)
    if args.design in DESIGNS:
        cfg = DESIGNS[args.design](args.layers, args.size, args.positions)
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
        args.size = cfg.get("architectures", [cfg.get("architecture", "?")])[0]
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
            "config": {"model": args.size + "-sizes" + (f" ({args.design.capitalize()})" if args.design in DESIGNS else ""),
                       "n_layer": cfg["n_layer"], "n_layer_full": SIZES[args.size][0],
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
