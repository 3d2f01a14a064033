"""A checkpoint's tokenizer, read from the model folder with the `tokenizers` library.

Rules of the reference's loader (engine/tokenizer.py:628-655): the tokenizer must name an
end-of-sequence token, and one without a padding token pads with that one.  The surface is
what the reference's entry points call (run.py:53,66-67, llm_engine.py:31-37): `encode`,
`decode`, `batch_decode`, `eos_token_id`, `bos_token_id`, `pad_token_id`, `len()`.  Only
files in the model folder are read (tokenizer.json for the vocabulary and rules;
tokenizer_config.json, special_tokens_map.json, generation_config.json and config.json
for which tokens are special); nothing is downloaded.  The engine itself needs no
tokenizer: prompts may be token ids.
"""

from __future__ import annotations

import json
from pathlib import Path


def _token_text(entry) -> str | None:
    """A special token as the config files write it: a string, or a dict with `content`."""
    if isinstance(entry, dict):
        entry = entry.get("content")
    return entry if isinstance(entry, str) else None


def _read_json(path: Path) -> dict:
    if not path.is_file():
        return {}
    data = json.loads(path.read_text())
    return data if isinstance(data, dict) else {}


class TextTokenizer:
    """Text to token ids and back, over a `tokenizers.Tokenizer`."""

    def __init__(self, core, *, eos_token_id, bos_token_id=None, pad_token_id=None):
        self.core = core
        self.eos_token_id, self.bos_token_id = eos_token_id, bos_token_id
        self.pad_token_id = pad_token_id

    def __len__(self) -> int:
        return self.core.get_vocab_size(with_added_tokens=True)

    def encode(self, text: str, add_special_tokens: bool = True) -> list[int]:
        return list(self.core.encode(text, add_special_tokens=add_special_tokens).ids)

    def decode(self, token_ids, skip_special_tokens: bool = True) -> str:
        return self.core.decode(list(token_ids), skip_special_tokens=skip_special_tokens)

    def batch_decode(self, sequences, skip_special_tokens: bool = True) -> list[str]:
        return self.core.decode_batch([list(s) for s in sequences],
                                      skip_special_tokens=skip_special_tokens)


def load_tokenizer(model_dir, *, set_none_pad_token_to_eos: bool = True) -> TextTokenizer:
    model_dir = Path(model_dir)
    if not (model_dir / "tokenizer.json").is_file():
        raise FileNotFoundError(
            f"no tokenizer.json in {model_dir}; pass token ids (--prompt-ids) instead of text")
    from tokenizers import Tokenizer

    core = Tokenizer.from_file(str(model_dir / "tokenizer.json"))
    named = {}
    for name in ("special_tokens_map.json", "tokenizer_config.json"):    # the later file wins
        named.update(_read_json(model_dir / name))
    ids = {}
    for role in ("eos", "bos", "pad"):
        text = _token_text(named.get(f"{role}_token"))
        ids[role] = core.token_to_id(text) if text is not None else None
        if text is not None and ids[role] is None:
            raise RuntimeError(f"{role}_token {text!r} is not in the tokenizer's vocabulary")
    if ids["eos"] is None:
        # no token named: the id that the generation or model configuration gives
        for name in ("generation_config.json", "config.json"):
            eos = _read_json(model_dir / name).get("eos_token_id")
            if isinstance(eos, list) and eos:
                eos = eos[0]
            if isinstance(eos, int) and core.id_to_token(eos) is not None:
                ids["eos"] = eos
                break
    if ids["eos"] is None:
        raise RuntimeError("Tokenizer without eos_token_id not supported.")
    if ids["pad"] is None and set_none_pad_token_to_eos:
        ids["pad"] = ids["eos"]
    return TextTokenizer(core, eos_token_id=ids["eos"], bos_token_id=ids["bos"],
                         pad_token_id=ids["pad"])


def describe(tokenizer) -> str:
    """One line for the log: class, size and the special tokens' ids."""
    return (f"{type(tokenizer).__name__} | size {len(tokenizer)} | "
            f"BOS {tokenizer.bos_token_id} | EOS {tokenizer.eos_token_id} | "
            f"PAD {tokenizer.pad_token_id}")
