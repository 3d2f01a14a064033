"""Decode and prefill throughput at the Qwen3-0.6B shape with random weights.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the engine (schedule, run, sample, postprocess) for a batch
of 8 requests with 512-token prompts; `value` is decoded tokens per second, counted from
the tokens the requests received in the timed steps.  The same line carries a 2,048-token
prefill, decode at batch 1, 64 and 256 and at longer contexts (`points`, with each
point's fraction of the HBM rate, mean context and step time beside it), the split of a
step into products and attention, a float32 decode point, and the decode step's fraction
of the HBM roofline.  Peaks are MI355X's published ones.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}


def make_engine(raw, dtype, layers, batch, max_len, budget, page_size, seed=0, model=None,
                eager=False):
    import torch
    from tokensprint_amd.config import Config
    from tokensprint_amd.engine.assemble import random_model
    from tokensprint_amd.engine.llm_engine import LLMEngine
    import tempfile
    if model is None:
        cfg = dict(raw)
        cfg["num_hidden_layers"] = layers
        _, model = random_model(cfg, seed, dtype, "cuda:0")
    pages = batch * (-(-max_len // page_size) + 1)
    config = Config(model=tempfile.gettempdir(), max_model_len=max_len, dtype=model.ctx.dtype,
                    kvcache_block_size=page_size, num_kvcache_blocks=pages,
                    max_num_seqs=max(batch, 1), max_num_batched_tokens=budget,
                    chunked_prefill=True, eos=-1, enforce_eager=eager)
    return model, LLMEngine(model, config)


def decode_points(batch, prompt_len, steps, warmup, context=4096):
    """Every decode measurement of a run: name -> (requests, prompt tokens, timed steps,
    warm-up steps, token budget of a step).  The first is the headline.  The same prompts
    and number of decoded tokens at batch 1 and 64; more requests than the captured decode
    kernels for few rows take (the library's products and norm kernels from 65 rows on) at
    256; and contexts of 2,048 and 4,096 tokens, reached by prompts that end 256 short of
    them."""
    points = {"headline": (batch, prompt_len, steps, warmup, 2048)}
    for b in (1, 64):
        points[f"decode_b{b}"] = (b, prompt_len, steps, warmup, 2048)
    points["decode_b256"] = (256, prompt_len, min(steps, 112), min(warmup, 16), 8192)
    for b in (8, 64):
        for ctx in (context // 2, context):
            points[f"decode_b{b}_ctx{ctx}"] = (b, ctx - 256, min(steps, 112), min(warmup, 16),
                                               8192)
    return points


def decode_lengths(batch, prompt_len, steps, warmup, budget):
    """(max_model_len, max_tokens) with which `decode_run` keeps every request alive to the
    end of the timed steps.  A request whose prompt is through decodes beside the others'
    prompt portions, one token a step, so the first one is ahead of the last by the
    number of steps the prompts take; nobody may reach a limit before the last timed step."""
    prefill_steps = -(-batch * prompt_len // budget) + batch
    max_tokens = prefill_steps + warmup + steps + 8
    return prompt_len + max_tokens + 1, max_tokens


def decode_run(engine, batch, prompt_len, steps, warmup, vocab, max_tokens):
    """Prefill `batch` prompts, then time exactly `steps` decode steps.  Returns (seconds,
    tokens decoded in them, mean over the timed steps of the tokens all live requests
    hold).  The decoded tokens are counted from the requests, and every request must be
    live and decoding from the first timed step to the last."""
    import torch
    from tokensprint_amd.config import SamplingParams
    g = torch.Generator().manual_seed(0)
    params = SamplingParams(temperature=0.0, max_tokens=max_tokens, ignore_eos=True)
    for _ in range(batch):
        engine.add_request(torch.randint(0, vocab, (prompt_len,), generator=g).tolist(), params)
    reqs = list(engine.requests.values())
    while any(r.num_completion_tokens == 0 for r in reqs):
        engine.step()                      # prefill portions until every request has a token
    for _ in range(warmup):
        engine.step()
    sync = torch.cuda.synchronize if torch.cuda.is_available() else (lambda: None)
    live0 = len(engine.scheduler.running)
    done0 = sum(r.num_completion_tokens for r in reqs)
    ctx0 = sum(len(r) for r in engine.scheduler.running)
    sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    sync()
    dt = time.perf_counter() - t0
    live1 = len(engine.scheduler.running)
    decoded = sum(r.num_completion_tokens for r in reqs) - done0
    ctx1 = sum(len(r) for r in engine.scheduler.running)
    if live0 != batch or live1 != batch or decoded != batch * steps:
        raise RuntimeError(
            f"decode run of {batch} requests: {live0} live before and {live1} after the timed "
            f"steps, {decoded} tokens decoded where {batch * steps} were expected")
    # drop the requests (one step may still be in flight: let it land first)
    sync()
    engine._flight = None
    for r in list(engine.scheduler.running):
        engine.scheduler.manager.free(r.cache)
    engine.scheduler.running.clear()
    engine.requests.clear()
    return dt, decoded, (ctx0 + ctx1) / 2.0


PRODUCTS = ("linear", "norm_linear", "linear_into_stream", "linear_silu_mul")
ATTENTION = ("attend", "paged_attention")


class Without:
    """The kernel provider with one kind of call made empty: products, or attention,
    return a block of zeros of the right shape and launch nothing.  A step captured this
    way holds the other kernels only, so its replay time is theirs."""

    def __init__(self, ops, kind):
        import torch
        self.ops, self.kind, self.torch = ops, kind, torch
        self.zeros = {}

    def _block(self, shape, dtype):
        key = (tuple(shape), dtype)
        if key not in self.zeros:
            self.zeros[key] = self.torch.zeros(*shape, dtype=dtype, device=self.ops.device)
        return self.zeros[key]

    def __enter__(self):
        ops, block = self.ops, self._block
        if self.kind == "attention":
            def attend(qkv, batch, table, cache, write_cache, *, num_heads, head_dim, **kw):
                return block((qkv.shape[0], num_heads, head_dim), qkv.dtype)

            def paged_attention(q, *args, **kw):
                return block(q.shape, q.dtype)
            ops.attend, ops.paged_attention = attend, paged_attention
        else:
            def linear(x, weight, out_dtype):
                return block((x.shape[0], weight.shape[0]), out_dtype)

            def linear_silu_mul(x, weight, out_dtype):
                return block((x.shape[0], weight.shape[0] // 2), out_dtype)

            def norm_linear(resid, delta, norm_weight, eps, weight, out_dtype, silu_mul=False):
                n = weight.shape[0] // 2 if silu_mul else weight.shape[0]
                return block((resid.shape[0], n), out_dtype), resid

            ops.linear, ops.linear_silu_mul, ops.norm_linear = linear, linear_silu_mul, norm_linear
            ops.linear_into_stream = lambda *a, **k: None
        return self

    def __exit__(self, *exc):
        for name in (ATTENTION if self.kind == "attention" else PRODUCTS):
            delattr(self.ops, name)              # the class's method shows again


def captured_seconds(runner, batch, reps=20):
    """Seconds per replay of `runner.run(batch)` captured as a graph."""
    import torch
    dev = runner.device
    side = torch.cuda.Stream(dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        runner.run(batch)
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        runner.run(batch)
    for _ in range(3):
        graph.replay()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        graph.replay()
    b.record()
    torch.cuda.synchronize(dev)
    return a.elapsed_time(b) * 1e-3 / reps


def step_split(model, page, entries_of, max_len):
    """(seconds of the whole step, of its products, of its attention) for the step that
    `entries_of(runner)` describes, each from a captured graph: the whole step, the step
    without attention, the step without products."""
    from tokensprint_amd.engine.runner import ModelRunner
    lengths = entries_of(None)
    pages = sum(-(-n // page) + 1 for n in lengths)
    runner = ModelRunner(model, page_size=page, num_pages=pages, num_slots=len(lengths))
    entries = entries_of(runner)
    width = [-(-max_len // page)] * len(runner.storage.groups)
    batch = runner.build(entries, width)
    batch.max_ctx_len = max_len
    whole = captured_seconds(runner, batch)
    with Without(model.ctx.ops, "attention"):
        batch.plans.clear()
        no_attention = captured_seconds(runner, batch)
    with Without(model.ctx.ops, "products"):
        batch.plans.clear()
        no_products = captured_seconds(runner, batch)
    batch.plans.clear()
    return whole, whole - no_products, whole - no_attention


def decode_entries(batch, context):
    """A decode step of `batch` requests that hold `context` tokens each."""
    from tokensprint_amd.engine.batch import StepEntry

    def make(runner):
        if runner is None:
            return [context + 1] * batch
        out = []
        for i in range(batch):
            rc = runner.manager.admit(i)
            runner.manager.extend(rc, context + 1)
            out.append(StepEntry(rc, [1], context, [0]))
        return out
    return make


def prefill_entries(tokens):
    from tokensprint_amd.engine.batch import StepEntry

    def make(runner):
        if runner is None:
            return [tokens]
        rc = runner.manager.admit(0)
        runner.manager.extend(rc, tokens)
        return [StepEntry(rc, [1] * tokens, 0, [tokens - 1])]
    return make


def prefill_run(engine, tokens, vocab, reps=5):
    import torch
    from tokensprint_amd.config import SamplingParams
    g = torch.Generator().manual_seed(1)
    times = []
    for _ in range(reps + 1):
        engine.add_request(torch.randint(0, vocab, (tokens,), generator=g).tolist(),
                           SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    times = sorted(times[1:])
    return times[len(times) // 2]


def cache_bytes(model, context, item) -> float:
    """Bytes of cache a decode step reads for one request that holds `context` tokens: of
    every run that owns a paged cache, keys and values of the tokens its mixer can see
    (all of them, or a window's)."""
    total = 0.0
    for need in model.cache_needs():
        if need is not None and hasattr(need, "num_kv_heads"):
            seen = context if need.window is None else min(context, need.window)
            total += 2 * need.num_kv_heads * need.head_dim * item * seen
    return total


def prefill_attention_flops(cfg, T) -> float:
    """Causal QK^T and PV of one layer for one prompt of T tokens."""
    return 2 * 2 * cfg["num_attention_heads"] * cfg["head_dim"] * T * (T + 1) / 2


def prefill_flops(cfg, layers, T) -> float:
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nq, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    per_token = 2 * H * (nq + 2 * nkv) * hd + 2 * nq * hd * H + 3 * 2 * H * I
    return layers * (per_token * T + prefill_attention_flops(cfg, T)) + 2 * H * V   # head: last token only


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=496)   # with the warmup: 512 tokens decoded
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--model", default="qwen3-0.6b")
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--context", type=int, default=4096,
                    help="the benchmark's context length: the long-context points decode at "
                         "half of it and at it")
    ap.add_argument("--skip-points", action="store_true", help="only the headline decode run")
    ap.add_argument("--skip-fp32", action="store_true", help="no float32 decode point")
    ap.add_argument("--only-prefill", action="store_true",
                    help="only the 2,048-token prefill (for profiling); prints its own line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import torch
    from tokensprint_amd.config import load_named_config

    raw = load_named_config(args.model)
    full_layers = raw["num_hidden_layers"]
    layers = args.layers or full_layers
    ctx_len, page = args.context, 16
    dt_name = "bf16" if args.dtype == "bfloat16" else "fp32"
    item = 2 if dt_name == "bf16" else 4
    vocab = raw["vocab_size"]

    if args.only_prefill:
        model, pre_engine = make_engine(raw, args.dtype, layers, 1, ctx_len, 2048, page)
        sec = prefill_run(pre_engine, 2048, vocab)
        print(json.dumps({"prefill_ms": round(sec * 1e3, 3), "tokens": 2048,
                          "tok_per_s": round(2048 / sec, 1)}))
        return 0
    plan = decode_points(args.batch, args.prompt_len, args.steps, args.warmup, ctx_len)
    if args.skip_points:
        plan = {"headline": plan["headline"]}
    model, results = None, {}
    for name, (b, prompt_len, steps, warmup, budget) in plan.items():
        max_len, max_tokens = decode_lengths(b, prompt_len, steps, warmup, budget)
        model, engine = make_engine(raw, args.dtype, layers, b, max_len, budget, page,
                                    model=model)
        if name == "headline":
            wbytes = model.step_weight_bytes()   # every weight a decode step reads, each once
        sec, decoded, held = decode_run(engine, b, prompt_len, steps, warmup, vocab, max_tokens)
        step_bytes = wbytes + cache_bytes(model, held / b, item) * b
        results[name] = {"tok_s": decoded / sec, "ms_step": sec / steps * 1e3,
                         "context": held / b, "gbs": step_bytes * steps / sec / 1e9}
        del engine
        torch.cuda.empty_cache()

    head = results["headline"]
    out = {
        "metric": f"decode tok/s at batch {args.batch} ({args.model} shape, "
                  f"{args.prompt_len}-token prompts)",
        "value": round(head["tok_s"], 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(head["ms_step"], 4),
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dt_name,
        "data": "synthetic: uniform random token ids, random weights N(0, 0.02) seed 0",
        "config": {
            "model": args.model, "global_batch": args.batch, "seq_len": ctx_len,
            "parallelism": "single-gpu", "layers": layers, "layers_of_model": full_layers,
            "hidden_size": raw["hidden_size"], "num_heads": raw["num_attention_heads"],
            "num_kv_heads": raw["num_key_value_heads"], "head_dim": raw["head_dim"],
            "intermediate_size": raw["intermediate_size"], "vocab_size": vocab,
            "tied_embeddings": raw["tie_word_embeddings"], "prompt_len": args.prompt_len,
            "page_size": page, "mean_context": round(head["context"], 1),
        },
        "roofline": {"bound": "hbm", "achieved": round(head["gbs"], 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(head["gbs"] / HBM_PEAK_GBS, 4)},
    }

    if not args.skip_points:
        # where the decode step's time goes, from captured steps with one kind of kernel
        # taken out: products against the weights they stream, attention against the cache
        def split(b, context, into, prefix=""):
            whole, t_products, t_attention = step_split(model, page, decode_entries(b, context),
                                                        ctx_len)
            into[prefix + "products_gbs"] = round(wbytes / t_products / 1e9, 1)
            into[prefix + "products_us"] = round(t_products * 1e6, 1)
            into[prefix + "attention_gbs"] = round(
                cache_bytes(model, context, item) * b / t_attention / 1e9, 1)
            into[prefix + "attention_us"] = round(t_attention * 1e6, 1)
            into[prefix + "step_us_without_host"] = round(whole * 1e6, 1)
        split(args.batch, int(round(head["context"])), out["roofline"])

        T = 2048
        _, pre_engine = make_engine(raw, args.dtype, layers, 1, ctx_len, T, page, model=model)
        sec = prefill_run(pre_engine, T, vocab)
        flops = prefill_flops(raw, layers, T)
        peak = MFMA_PEAK_TFLOPS[dt_name] * 1e12
        out["prefill"] = {"value": round(T / sec, 1), "tokens": T, "ms": round(sec * 1e3, 3),
                          "frac": round(flops / sec / peak, 4)}
        attn_flops = layers * prefill_attention_flops(raw, T)
        _, t_products, t_attention = step_split(model, page, prefill_entries(T), ctx_len)
        out["prefill"]["products_tflops"] = round((flops - attn_flops) / t_products / 1e12, 1)
        out["prefill"]["products_us"] = round(t_products * 1e6, 1)
        out["prefill"]["attention_tflops"] = round(attn_flops / t_attention / 1e12, 1)
        out["prefill"]["attention_us"] = round(t_attention * 1e6, 1)
        del pre_engine
        torch.cuda.empty_cache()
        names = [n for n in results if n != "headline"]
        out["points"] = {n: round(results[n]["tok_s"], 1) for n in names}
        # of every point: its fraction of the HBM rate (weights once and the live requests'
        # cache, over its measured step), the mean context it was measured at, its step
        out["points_frac"] = {n: round(results[n]["gbs"] / HBM_PEAK_GBS, 4) for n in names}
        out["points_context"] = {n: round(results[n]["context"], 1) for n in names}
        out["points_ms_per_step"] = {n: round(results[n]["ms_step"], 4) for n in names}
        out["points_split"] = {}
        for n in ("decode_b1", "decode_b64"):
            split(plan[n][0], int(round(results[n]["context"])), out["points_split"], n + "_")
        if dt_name == "bf16" and not args.skip_fp32:
            # the true 32-bit path at the headline's batch: its own weights, cache and kernels
            del model
            torch.cuda.empty_cache()
            b, prompt_len, steps, warmup, budget = plan["headline"]
            steps, warmup = min(steps, 48), min(warmup, 4)
            max_len, max_tokens = decode_lengths(b, prompt_len, steps, warmup, budget)
            model32, engine = make_engine(raw, "float32", layers, b, max_len, budget, page)
            sec, decoded, held = decode_run(engine, b, prompt_len, steps, warmup, vocab,
                                            max_tokens)
            bytes32 = model32.step_weight_bytes() + cache_bytes(model32, held / b, 4) * b
            out["points"][f"decode_b{b}_fp32"] = round(decoded / sec, 1)
            out["points_frac"][f"decode_b{b}_fp32"] = round(
                bytes32 * steps / sec / 1e9 / HBM_PEAK_GBS, 4)
            out["points_context"][f"decode_b{b}_fp32"] = round(held / b, 1)
            out["points_ms_per_step"][f"decode_b{b}_fp32"] = round(sec / steps * 1e3, 4)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
