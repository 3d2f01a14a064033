"""Loading a checkpoint's tokenizer, with the reference's rules
(engine/tokenizer.py:628-655): it must name an end-of-sequence token, and a tokenizer
without a padding token pads with that one.  Only files in the model folder are read;
nothing is downloaded.  The engine itself needs no tokenizer: prompts may be token ids.
"""

from __future__ import annotations

from pathlib import Path


def load_tokenizer(model_dir, *, use_fast: bool = True, set_none_pad_token_to_eos: bool = True):
    model_dir = Path(model_dir)
    if not any((model_dir / name).is_file()
               for name in ("tokenizer.json", "tokenizer_config.json", "tokenizer.model")):
        raise FileNotFoundError(
            f"no tokenizer files in {model_dir}; pass token ids (--prompt-ids) instead of text")
    from transformers import AutoTokenizer      # imported late: it takes seconds

    tokenizer = AutoTokenizer.from_pretrained(str(model_dir), use_fast=use_fast,
                                              local_files_only=True)
    if tokenizer.eos_token_id is None:
        raise RuntimeError("Tokenizer without eos_token_id not supported.")
    if tokenizer.pad_token_id is None and set_none_pad_token_to_eos:
        tokenizer.pad_token = tokenizer.eos_token
    return tokenizer


def describe(tokenizer) -> str:
    """One line for the log: class, size and the special tokens' ids."""
    return (f"{type(tokenizer).__name__} | size {len(tokenizer)} | "
            f"BOS {tokenizer.bos_token_id} | EOS {tokenizer.eos_token_id} | "
            f"PAD {tokenizer.pad_token_id}")
