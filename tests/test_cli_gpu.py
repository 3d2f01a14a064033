"""The command-line programs, run as a user runs them (child processes on the GPU):
run.py with a named tiny model and random weights against the plain implementation, with
the cache pool sized from free memory; benchmark.py; model_registry.py."""

import json
import os
import re
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from helpers import TINY_A, TINY_B, random_prompt, write_word_tokenizer
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


def config_json(tmp_path, cfg):
    path = tmp_path / "config_for_random_weights.json"
    path.write_text(json.dumps(cfg))
    return path


def run_program(args, timeout=300):
    env = dict(os.environ, PYTHONUNBUFFERED="1")
    proc = subprocess.run([sys.executable, *map(str, args)], cwd=ROOT, env=env, text=True,
                          capture_output=True, timeout=timeout)
    assert proc.returncode == 0, f"{args}\n{proc.stdout[-2000:]}\n{proc.stderr[-4000:]}"
    return proc


@pytest.mark.parametrize("dtype,extra", [
    ("float32", []),                                        # --num-pages stays -1: measured
    ("float32", ["--num-pages", "40", "--chunked-prefill", "True",
                 "--max-num-batched-tokens", "8", "--enforce-eager", "True"]),
])
def test_run_py_generates_the_plain_tokens(gpu_device, tmp_path, dtype, extra):
    prompt = random_prompt(19, 389, 5)
    model_dir = tmp_path / "tiny-b"
    proc = run_program(["run.py", "--config-json", config_json(tmp_path, TINY_B),
                        "--random-weights", "1",
                        "--model-dir", model_dir, "--dtype", dtype, "--temperature", "0",
                        "--max-tokens", "14", "--ignore-eos", "True", "--max-num-seqs", "16",
                        "--prompt-ids", ",".join(map(str, prompt)), *extra])
    got = json.loads(proc.stdout.strip().splitlines()[-1])
    pcfg, w = plain.read_model_dir(model_dir)       # the folder run.py wrote and loaded
    assert got == plain.greedy_generate(pcfg, w, prompt, 14)
    if not extra:
        pages = re.search(r"key/value cache: (\d+) pages", proc.stderr)
        assert pages and int(pages.group(1)) >= 16, proc.stderr[-2000:]
        assert "largest step" in proc.stderr


def test_run_py_bfloat16_runs_and_samples(gpu_device, tmp_path):
    prompt = random_prompt(40, 256, 6)
    out = []
    for _ in range(2):
        proc = run_program(["run.py", "--config-json", config_json(tmp_path, TINY_A),
                            "--random-weights", "0",
                            "--model-dir", tmp_path / "tiny-a", "--temperature", "0.8",
                            "--max-tokens", "9", "--ignore-eos", "True", "--max-num-seqs", "8",
                            "--page-size", "4", "--seed", "11",
                            "--prompt-ids", ",".join(map(str, prompt))])
        out.append(json.loads(proc.stdout.strip().splitlines()[-1]))
    assert len(out[0]) == 9 and all(0 <= t < 256 for t in out[0])
    assert out[0] == out[1]                         # a seeded draw: the same tokens again


def test_run_py_with_a_text_prompt(gpu_device, tmp_path):
    """The text path (run.py:42-68 of the reference): the folder's tokenizer encodes the
    prompt, its end-of-sequence token ends the request, and what is printed is its
    decoding of the completion without special tokens."""
    from tokensprint_amd.weights import write_random_model
    model_dir = tmp_path / "tiny-b-with-tokenizer"
    write_random_model(model_dir, TINY_B, 1, torch.float32)
    pcfg, w = plain.read_model_dir(model_dir)
    prompt = [t or 1 for t in random_prompt(19, 389, 5)]          # id 0 is the unknown word
    completion = plain.greedy_generate(pcfg, w, prompt, 14)
    # the end-of-sequence token: one the greedy completion meets for the first time after
    # a few tokens, so that the request has to stop there
    stop = next(k for k in range(3, 14) if completion[k] not in completion[:k] + [0])
    eos = completion[stop]
    tok = write_word_tokenizer(model_dir, TINY_B["vocab_size"], eos_id=eos)
    text = " ".join(tok.id_to_token(t) for t in prompt)
    assert tok.encode(text).ids == prompt
    common = ["run.py", "--model-dir", model_dir, "--dtype", "float32", "--temperature", "0",
              "--max-tokens", "14", "--max-num-seqs", "16", "--prompt", text]
    proc = run_program(common)
    assert proc.stdout.strip().splitlines()[-1] == tok.decode(completion[:stop])
    assert f"EOS {eos}" in proc.stderr and "TextTokenizer" in proc.stderr
    proc = run_program(common + ["--ignore-eos", "True"])
    assert proc.stdout.strip().splitlines()[-1] == tok.decode(completion)   # skips the special one
    assert len(tok.decode(completion).split()) == sum(t not in (0, eos) for t in completion)


def test_benchmark_py(gpu_device, tmp_path):
    proc = run_program(["benchmark.py", "--config-json", config_json(tmp_path, TINY_B),
                        "--num-seqs", "8",
                        "--max-input-len", "120", "--max-output-len", "120",
                        "--max-num-seqs", "8", "--use-tqdm", "False"])
    line = [ln for ln in proc.stdout.splitlines() if "Throughput" in ln][-1]
    m = re.search(r"Total: (\d+)tok, Time: ([\d.]+)s, Throughput: ([\d.]+)tok/s", line)
    assert m and int(m.group(1)) >= 8 * 100 and float(m.group(3)) > 0, line


def test_benchmark_py_with_a_pool_that_forces_preemption(gpu_device, tmp_path):
    proc = run_program(["benchmark.py", "--config-json", config_json(tmp_path, TINY_B),
                        "--num-seqs", "6",
                        "--min-input-len", "100", "--max-input-len", "100",
                        "--min-output-len", "60", "--max-output-len", "60",
                        "--max-num-seqs", "6", "--num-pages", "30", "--use-tqdm", "False",
                        "--max-num-batched-tokens", "64"])
    line = [ln for ln in proc.stdout.splitlines() if "Throughput" in ln][-1]
    assert "Total: 360tok" in line and int(re.search(r"preemptions: (\d+)", line).group(1)) > 0


def test_model_registry_py():
    proc = run_program(["model_registry.py"])
    assert "qwen:\n  - qwen3-0.6b (qwen/qwen3-0.6b)" in proc.stdout
    assert "tiny" not in proc.stdout               # test configurations are no presets
    assert "Qwen3ForCausalLM" in proc.stdout
