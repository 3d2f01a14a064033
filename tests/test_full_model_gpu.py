"""The Qwen3-0.6B configuration unchanged (engine/models/qwen/_archs.py:92-125 of the
reference: 28 layers, a vocabulary of 151,936, tied head) with random weights, in
float32 and in bfloat16, against the plain implementation on the CPU: what 28 layers of
rounding add up to, and the output head at its real width."""

import pytest
import torch

import drives
from helpers import random_prompt
from plain import qwen3_plain as plain
from tokensprint_amd.config import load_named_config
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

TOL = {torch.float32: (1e-4, 2e-5), torch.bfloat16: (3e-2, 3e-2)}
PAGE = 16
LONG = 700


@pytest.fixture(scope="module", params=[torch.float32, torch.bfloat16],
                ids=lambda d: str(d).split(".")[-1])
def setup(request, tmp_path_factory, gpu_device):
    dtype = request.param
    cfg = load_named_config("qwen3-0.6b")
    assert (cfg["num_hidden_layers"], cfg["vocab_size"]) == (28, 151936)
    d = tmp_path_factory.mktemp("qwen3-0.6b")
    write_random_model(d, cfg, 0, dtype, device=gpu_device)     # drawn on the GPU: seconds
    pcfg, w = plain.read_model_dir(d)          # the same (rounded) weights, held in float32
    requests = {f"r{i}": random_prompt(n, cfg["vocab_size"], 300 + i)
                for i, n in enumerate([5, 40, 100])}
    ref = {rid: plain.forward_logits(pcfg, w, t) for rid, t in requests.items()}
    # one prompt long enough for the kernels that only steps of many rows take (the
    # LDS-tiled products with the residual add and the norm inside)
    long_prompt = {"long": random_prompt(LONG, cfg["vocab_size"], 310)}
    long_ref = {rid: plain.forward_logits(pcfg, w, t) for rid, t in long_prompt.items()}
    del w
    _, model = load_model(d, dtype, gpu_device)
    model.long_prompt, model.long_ref = long_prompt, long_ref
    yield model, requests, ref, TOL[dtype]
    del model
    torch.cuda.empty_cache()


def test_whole(setup):
    model, requests, ref, (rtol, atol) = setup
    runner = ModelRunner(model, page_size=PAGE, num_pages=112 // PAGE, num_slots=4)
    drives.compare(drives.drive_whole(runner, requests), ref, rtol, atol)


def test_prefill_then_decode(setup):
    model, requests, ref, (rtol, atol) = setup
    runner = ModelRunner(model, page_size=PAGE, num_pages=112 // PAGE, num_slots=4)
    drives.compare(drives.drive_prefill_then_decode(runner, requests), ref, rtol, atol)


def test_mixed_with_page_reuse(setup):
    model, requests, ref, (rtol, atol) = setup
    # ten pages where the three requests need 1 + 3 + 7: the shortest one's page is used again
    runner = ModelRunner(model, page_size=PAGE, num_pages=10, num_slots=4)
    drives.compare(drives.drive_mixed(runner, requests), ref, rtol, atol)
    assert all(pool.num_used == 0 for pool in runner.manager.pools)


def test_long_prompt_whole_and_in_portions(setup):
    """700 tokens in one step (the products of many rows, fused with the stream's add and
    norm where the provider does that) and in portions of 300 and 400 (the separate
    kernels), both against the plain implementation."""
    model, _, _, (rtol, atol) = setup
    runner = ModelRunner(model, page_size=PAGE, num_pages=(LONG + PAGE - 1) // PAGE + 1, num_slots=4)
    ref = model.long_ref
    drives.compare(drives.drive_whole(runner, model.long_prompt), ref, rtol, atol)
    drives.compare(drives.drive_portions(runner, model.long_prompt, sizes=(300, 400)), ref, rtol, atol)
