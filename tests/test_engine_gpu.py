"""The engine with the HIP kernels on the GPU against the plain implementation: every
way of cutting requests into steps, in float32 and in bfloat16, for the tiny
configurations.  Tolerances are fixed by the arithmetic (float32: a few units of
rounding over the depth; bfloat16: activations rounded to 8 bits between kernels), not
fitted to results."""

import pytest
import torch

import drives
from helpers import TINY, random_prompt
from plain import qwen3_plain as plain
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

TOL = {torch.float32: (1e-4, 2e-5), torch.bfloat16: (3e-2, 3e-2)}


@pytest.fixture(scope="module", params=[(n, d) for n in sorted(TINY)
                                        for d in (torch.float32, torch.bfloat16)],
                ids=lambda p: f"{p[0]}-{str(p[1]).split('.')[-1]}")
def setup(request, tmp_path_factory, gpu_device):
    name, dtype = request.param
    cfg, seed, page = TINY[name]
    d = tmp_path_factory.mktemp(f"tiny{name}")
    write_random_model(d, cfg, seed, dtype)
    pcfg, w = plain.read_model_dir(d)          # the same (rounded) weights, held in float32
    _, model = load_model(d, dtype, gpu_device)
    lengths = [5, 11, 17, 40, 64, 1, 23, 100]
    requests = {f"r{i}": random_prompt(n, cfg["vocab_size"], 100 + i)
                for i, n in enumerate(lengths)}
    ref = {rid: plain.forward_logits(pcfg, w, t) for rid, t in requests.items()}
    return model, page, requests, ref, TOL[dtype]


def runner_for(model, page, num_pages):
    return ModelRunner(model, page_size=page, num_pages=num_pages, num_slots=4)


def test_whole(setup):
    model, page, requests, ref, (rtol, atol) = setup
    drives.compare(drives.drive_whole(runner_for(model, page, 128 // page), requests),
                   ref, rtol, atol)


def test_prefill_then_decode(setup):
    model, page, requests, ref, (rtol, atol) = setup
    drives.compare(drives.drive_prefill_then_decode(runner_for(model, page, 128 // page),
                                                    requests), ref, rtol, atol)


def test_portions(setup):
    model, page, requests, ref, (rtol, atol) = setup
    drives.compare(drives.drive_portions(runner_for(model, page, 128 // page), requests),
                   ref, rtol, atol)


def test_mixed_with_page_reuse(setup):
    model, page, requests, ref, (rtol, atol) = setup
    runner = runner_for(model, page, 224 // page)      # 261 tokens in all: pages are reused
    drives.compare(drives.drive_mixed(runner, requests), ref, rtol, atol)
    assert all(pool.num_used == 0 for pool in runner.manager.pools)
