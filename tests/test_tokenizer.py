"""The tokenizer loader's rules (engine/tokenizer.py:628-655 of the reference: an
end-of-sequence token is required, padding falls back to it) and the surface the entry
points use, over a word-level tokenizer written by the test."""

import json

import pytest

from helpers import write_word_tokenizer
from tokensprint_amd.tokenizer import describe, load_tokenizer


def test_encode_decode_and_special_ids(tmp_path):
    write_word_tokenizer(tmp_path, 50, eos_id=7)
    tok = load_tokenizer(tmp_path)
    assert len(tok) == 50
    assert tok.eos_token_id == 7 and tok.bos_token_id is None
    assert tok.pad_token_id == 7                      # no padding token: the end of sequence
    assert tok.encode("w5 w17  w3\nw49", add_special_tokens=True) == [5, 17, 3, 49]
    assert tok.encode("w5 nonsense") == [5, 0]
    assert tok.decode([5, 7, 17]) == "w5 w17"          # special tokens are skipped
    assert tok.decode([5, 7, 17], skip_special_tokens=False) == "w5 <eos> w17"
    assert tok.batch_decode([[1, 2], [7, 3]]) == ["w1 w2", "w3"]
    assert "EOS 7" in describe(tok) and "size 50" in describe(tok)


def test_a_padding_token_of_its_own_is_kept(tmp_path):
    write_word_tokenizer(tmp_path, 50, eos_id=7, pad_id=9)
    tok = load_tokenizer(tmp_path)
    assert (tok.eos_token_id, tok.pad_token_id) == (7, 9)
    assert load_tokenizer(tmp_path, set_none_pad_token_to_eos=False).pad_token_id == 9


def test_without_an_end_of_sequence_token_it_refuses(tmp_path):
    write_word_tokenizer(tmp_path, 50, name_eos=False)
    with pytest.raises(RuntimeError, match="eos_token_id"):
        load_tokenizer(tmp_path)
    # the id that config.json gives serves where no file names the token
    (tmp_path / "config.json").write_text(json.dumps({"eos_token_id": [11, 12]}))
    tok = load_tokenizer(tmp_path, set_none_pad_token_to_eos=False)
    assert tok.eos_token_id == 11 and tok.pad_token_id is None


def test_a_named_token_that_the_vocabulary_lacks(tmp_path):
    write_word_tokenizer(tmp_path, 50)
    (tmp_path / "tokenizer_config.json").write_text(json.dumps({"eos_token": "<|end|>"}))
    with pytest.raises(RuntimeError, match="not in the tokenizer's vocabulary"):
        load_tokenizer(tmp_path)


def test_no_tokenizer_files(tmp_path):
    with pytest.raises(FileNotFoundError, match="prompt-ids"):
        load_tokenizer(tmp_path)
