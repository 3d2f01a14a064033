"""The engine's cache manager, batch builder and step function on the CPU, with the
plain torch kernel references standing in for the HIP kernels: every way of cutting
requests into steps gives the plain implementation's logits (float32)."""

import pytest
import torch

import drives
from helpers import TINY, random_prompt
from kernel_refs import TorchOps
from plain import qwen3_plain as plain
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.weights import write_random_model


@pytest.fixture(scope="module", params=sorted(TINY))
def setup(request, tmp_path_factory):
    cfg, seed, page = TINY[request.param]
    d = tmp_path_factory.mktemp(f"tiny{request.param}")
    write_random_model(d, cfg, seed, torch.float32)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    lengths = [5, 11, 17, 40, 64, 1, 23]
    requests = {f"r{i}": random_prompt(n, cfg["vocab_size"], 100 + i)
                for i, n in enumerate(lengths)}
    ref = {rid: plain.forward_logits(pcfg, w, t) for rid, t in requests.items()}
    return model, page, requests, ref


def runner_for(model, page, num_pages):
    return ModelRunner(model, page_size=page, num_pages=num_pages, num_slots=4)


def test_whole(setup):
    model, page, requests, ref = setup
    drives.compare(drives.drive_whole(runner_for(model, page, 64 // page + 1), requests),
                   ref, 1e-4, 2e-5)


def test_prefill_then_decode(setup):
    model, page, requests, ref = setup
    drives.compare(drives.drive_prefill_then_decode(runner_for(model, page, 64 // page + 1),
                                                    requests), ref, 1e-4, 2e-5)


def test_portions(setup):
    model, page, requests, ref = setup
    drives.compare(drives.drive_portions(runner_for(model, page, 64 // page + 1), requests),
                   ref, 1e-4, 2e-5)


def test_mixed_with_page_reuse(setup):
    model, page, requests, ref = setup
    # pages for 160 tokens: less than the 161 tokens of all requests, so pages are reused
    runner = runner_for(model, page, 160 // page)
    drives.compare(drives.drive_mixed(runner, requests), ref, 1e-4, 2e-5)
    assert all(pool.num_used == 0 for pool in runner.manager.pools)


def test_preempted_and_recomputed(setup):
    model, page, requests, ref = setup
    runner = runner_for(model, page, 160 // page)
    drives.compare(drives.drive_preempted(runner, requests), ref, 1e-4, 2e-5)
    assert all(pool.num_used == 0 for pool in runner.manager.pools)
