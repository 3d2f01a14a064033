"""Single-prompt command line, in the manner of the reference's run.py:25-72.

Same options with the same meanings (--model-name, --cache-dir, --prompt, --max-tokens,
--temperature, --enforce-eager; booleans take a value, `--enforce-eager True`, as the
reference's FlagConversionOff does), plus what an engine without network needs:
--model-dir, --dtype, --random-weights SEED (for --model-name, or for the config.json that
--config-json names), --prompt-ids, and the cache and scheduler knobs of the engine
configuration.
"""

from __future__ import annotations

import argparse
import json
import logging
import tempfile
from pathlib import Path

logging.basicConfig(level=logging.INFO,
                    format="%(asctime)s %(levelname)s %(name)s: %(message)s", force=True)
log = logging.getLogger("run")


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
    ap.add_argument("--cache-dir", type=Path, default=Path("./local_data"))
    ap.add_argument("--prompt", default="Tell me a long story about transformers.")
    ap.add_argument("--max-tokens", type=int, default=1024)
    ap.add_argument("--temperature", type=float, default=0.8)
    ap.add_argument("--enforce-eager", type=_bool, default=False)
    ap.add_argument("--model-dir", type=Path, default=None,
                    help="model folder; default <cache-dir>/<model name>")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                    help="write a random-weights folder for --model-name and run that")
    ap.add_argument("--config-json", type=Path, default=None,
                    help="with --random-weights: this config.json instead of --model-name's")
    ap.add_argument("--prompt-ids", default=None,
                    help="comma-separated token ids instead of --prompt (no tokenizer needed)")
    ap.add_argument("--cast-weights", type=_bool, default=False,
                    help="bfloat16 run: round matrices the checkpoint stores in 32-bit to "
                         "bfloat16 (default: they stay 32-bit, on the float32 kernels)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--num-pages", type=int, default=-1)
    ap.add_argument("--max-num-batched-tokens", type=int, default=16384)
    ap.add_argument("--max-num-seqs", type=int, default=512)
    ap.add_argument("--max-model-len", type=int, default=None)
    ap.add_argument("--chunked-prefill", type=_bool, default=False)
    ap.add_argument("--prefix-caching", type=_bool, default=False,
                    help="share cached full pages between requests with equal prefixes")
    ap.add_argument("--ignore-eos", type=_bool, default=False)
    ap.add_argument("--seed", type=int, default=0)
    return ap.parse_args(argv)


def main(args) -> None:
    import torch

    from tokensprint_amd.config import (Config, SamplingParams, get_model_repo_id,
                                        load_named_config)
    from tokensprint_amd.engine.assemble import load_model, parse_dtype
    from tokensprint_amd.engine.llm_engine import LLMEngine
    from tokensprint_amd.weights import write_random_model

    if not torch.cuda.is_available():
        raise RuntimeError("A GPU is required: the engine has no CPU path.")
    dtype = parse_dtype(args.dtype)
    model_dir = args.model_dir
    if args.random_weights is not None:
        model_dir = model_dir or Path(tempfile.mkdtemp(prefix="tokensprint_random_"))
        raw = json.loads(args.config_json.read_text()) if args.config_json is not None \
            else load_named_config(args.model_name)
        write_random_model(model_dir, raw, args.random_weights, dtype)
    elif args.config_json is not None:
        raise ValueError("--config-json describes random weights: give --random-weights SEED")
    elif model_dir is None:
        model_dir = args.cache_dir / get_model_repo_id(args.model_name).split("/")[-1]
    _, model = load_model(model_dir, dtype, "cuda:0", cast_32bit=args.cast_weights)
    spec = model.spec           # sizes and the end-of-sequence token come from the model as
                                # built, whatever architecture config.json named

    tokenizer = None
    if args.prompt_ids is None:
        from tokensprint_amd.tokenizer import describe, load_tokenizer
        tokenizer = load_tokenizer(model_dir)
        log.info("tokenizer: %s", describe(tokenizer))
        prompt = args.prompt
    else:
        prompt = [int(t) for t in args.prompt_ids.split(",")]
    # end of sequence: the tokenizer's, as the reference's run.py:53; without a tokenizer
    # the one config.json names (ModelSpec.eos_token_id), else none
    if tokenizer is not None:
        eos = tokenizer.eos_token_id
    else:
        eos = spec.eos_token_id if spec.eos_token_id is not None else -1

    config = Config(
        model=str(model_dir), max_model_len=args.max_model_len or int(spec.max_position),
        eos=eos, dtype=dtype, enforce_eager=args.enforce_eager,
        kvcache_block_size=args.page_size, num_kvcache_blocks=args.num_pages,
        max_num_batched_tokens=args.max_num_batched_tokens, max_num_seqs=args.max_num_seqs,
        chunked_prefill=args.chunked_prefill, seed=args.seed,
        enable_prefix_caching=args.prefix_caching)
    engine = LLMEngine(model=model, config=config, tokenizer=tokenizer)
    params = SamplingParams(temperature=args.temperature, max_tokens=args.max_tokens,
                            ignore_eos=args.ignore_eos, seed=args.seed)
    outputs = engine.generate([prompt], params)
    if tokenizer is not None:
        print(tokenizer.batch_decode(outputs, skip_special_tokens=True)[0])
    else:
        print(json.dumps(outputs[0]))


if __name__ == "__main__":
    main(parse_args())
