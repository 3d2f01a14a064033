"""Throughput harness in the manner of the reference's benchmark.py:23-249: a seeded
synthetic workload of token-id prompts with random prompt and output lengths, one
warm-up request, then output tokens divided by wall time with a device synchronisation
on both sides.  Options keep the reference's names and meanings (booleans take a value:
`--use-tqdm False`); the comparison backend of the reference is not part of this engine.
Weights are random (of --model-name's configuration, or of the config.json that
--config-json names) unless --model-dir names a checkpoint folder.
"""

from __future__ import annotations

import argparse
import json
import tempfile
import time
from pathlib import Path
from random import randint, seed


def _bool(text: str) -> bool:
    if text.lower() in ("true", "1", "yes"):
        return True
    if text.lower() in ("false", "0", "no"):
        return False
    raise argparse.ArgumentTypeError(f"expected True or False, got {text!r}")


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model-name", default="qwen/qwen3-0.6b")
    ap.add_argument("--model-dir", type=Path, default=None)
    ap.add_argument("--config-json", type=Path, default=None,
                    help="random weights of this config.json instead of --model-name's")
    ap.add_argument("--num-seqs", type=int, default=256)
    ap.add_argument("--max-input-len", type=int, default=1024)
    ap.add_argument("--max-output-len", type=int, default=1024)
    ap.add_argument("--min-input-len", type=int, default=100,
                    help="prompt lengths are uniform in [min, max]; equal values fix them")
    ap.add_argument("--min-output-len", type=int, default=100)
    ap.add_argument("--max-model-len", type=int, default=None)
    ap.add_argument("--enforce-eager", type=_bool, default=False)
    ap.add_argument("--chunked-prefill", type=_bool, default=True)
    ap.add_argument("--max-num-batched-tokens", type=int, default=8192)
    ap.add_argument("--max-num-seqs", type=int, default=256)
    ap.add_argument("--use-tqdm", type=_bool, default=True)
    ap.add_argument("--max-prompt-token-id", type=int, default=10000)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--cast-weights", type=_bool, default=False,
                    help="with --model-dir, bfloat16: round 32-bit matrices to bfloat16")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--num-pages", type=int, default=-1)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers (random weights only)")
    ap.add_argument("--decode-ahead", type=_bool, default=True,
                    help="launch decode steps before the last one's tokens are read")
    return ap.parse_args(argv)


def make_workload(args):
    """The reference's synthetic workload (benchmark.py:54-63): per request a prompt of
    uniformly random token ids and length, and a uniformly random number of tokens to
    generate; the lower bounds, fixed at 100 there, are options here."""
    lo_in, lo_out = min(args.min_input_len, args.max_input_len), \
        min(args.min_output_len, args.max_output_len)
    prompts = []
    for _ in range(args.num_seqs):
        length = randint(lo_in, args.max_input_len)
        prompts.append([randint(0, args.max_prompt_token_id) for _ in range(length)])
    return prompts, [randint(lo_out, args.max_output_len) for _ in range(args.num_seqs)]


def main(args) -> None:
    import torch

    from tokensprint_amd.config import Config, SamplingParams, load_named_config
    from tokensprint_amd.engine.assemble import load_model, random_model
    from tokensprint_amd.engine.llm_engine import LLMEngine

    seed(0)
    prompts, output_lens = make_workload(args)
    if args.model_dir is not None:
        _, model = load_model(args.model_dir, args.dtype, "cuda:0", cast_32bit=args.cast_weights)
        model_dir = str(args.model_dir)
    else:
        raw = json.loads(args.config_json.read_text()) if args.config_json is not None \
            else load_named_config(args.model_name)
        if args.layers:
            raw["num_hidden_layers"] = args.layers
        _, model = random_model(raw, 0, args.dtype, "cuda:0")
        model_dir = tempfile.gettempdir()
    spec = model.spec
    max_model_len = args.max_model_len or int(spec.max_position)
    if max_model_len > spec.max_position:
        raise ValueError(f"max_model_len cannot exceed the model's {spec.max_position}")
    limit = min(args.max_prompt_token_id, spec.vocab_size - 1)
    prompts = [[min(t, limit) for t in p] for p in prompts]
    llm = LLMEngine(model, Config(
        model=model_dir, enforce_eager=args.enforce_eager, max_model_len=max_model_len,
        max_num_batched_tokens=args.max_num_batched_tokens, max_num_seqs=args.max_num_seqs,
        chunked_prefill=args.chunked_prefill, eos=-1, dtype=model.ctx.dtype,
        kvcache_block_size=args.page_size, num_kvcache_blocks=args.num_pages,
        decode_ahead=args.decode_ahead))
    params = [SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=n) for n in output_lens]
    llm.generate([[1, 2, 3]], SamplingParams(max_tokens=8, ignore_eos=True), use_tqdm=False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    llm.generate(prompts, params, use_tqdm=args.use_tqdm)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    total = sum(output_lens)
    prompt_tokens = sum(len(p) for p in prompts)
    print(f"[tokensprint_amd] Total: {total}tok, Time: {elapsed:.2f}s, "
          f"Throughput: {total / elapsed:.2f}tok/s, prompt tokens: {prompt_tokens}, "
          f"pages: {llm.config.num_kvcache_blocks}, preemptions: {llm.scheduler.num_preemptions}")


if __name__ == "__main__":
    main(parse_args())
