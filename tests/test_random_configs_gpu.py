"""Randomly drawn tiny configurations through every drive on the GPU, in float32 and
bfloat16, against the plain implementation: head sizes from 16 to 256, any grouping,
widths and vocabularies that are no power of two, windows, page sizes 16 to 64.  The
draws are seeded, so a run is repeatable; what they are for is the sizes nobody thought of."""

import random

import pytest
import torch

import drives
from helpers import qwen3_config, random_prompt
from plain import qwen3_plain as plain
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

TOL = {torch.float32: (1e-4, 2e-5), torch.bfloat16: (3e-2, 3e-2)}


def draw(case):
    rnd = random.Random(case)
    hd = rnd.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256])
    kv = rnd.choice([1, 2, 3, 4])
    group = rnd.choice([1, 2, 3, 4, 5, 8, 16, 20])
    layers = rnd.choice([1, 2, 3])
    window = rnd.choice([None, None, 5, 24, 70])
    layer_types = None
    if window is not None:
        layer_types = [rnd.choice(["full_attention", "sliding_attention"]) for _ in range(layers)]
        if "sliding_attention" not in layer_types:
            layer_types[0] = "sliding_attention"
    cfg = qwen3_config(hidden=rnd.choice([40, 64, 72, 100, 128, 136, 200, 256, 520]),
                       layers=layers, heads=kv * group, kv_heads=kv, head_dim=hd,
                       inter=rnd.choice([24, 56, 96, 130, 264, 520]),
                       vocab=rnd.choice([97, 256, 1000, 1031, 20001]),
                       eps=rnd.choice([1e-6, 1e-5]), theta=rnd.choice([1e4, 1e6]),
                       tied=rnd.random() < 0.5, max_pos=256, window=window,
                       layer_types=layer_types)
    return cfg, rnd.choice([16, 16, 32, 64])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("case", range(12))
def test_a_drawn_configuration(case, dtype, tmp_path, gpu_device):
    cfg, page = draw(case)
    write_random_model(tmp_path, cfg, case, dtype)
    pcfg, w = plain.read_model_dir(tmp_path)
    _, model = load_model(tmp_path, dtype, gpu_device)
    lengths = [5, 17, 40, 64, 1, 100, 130]
    requests = {f"r{i}": random_prompt(n, cfg["vocab_size"], 100 + i)
                for i, n in enumerate(lengths)}
    ref = {rid: plain.forward_logits(pcfg, w, t) for rid, t in requests.items()}
    rtol, atol = TOL[dtype]

    def runner(pages, **kw):
        return ModelRunner(model, page_size=page, num_pages=pages, num_slots=4, **kw)

    roomy = 192 // page + 4
    drives.compare(drives.drive_whole(runner(roomy), requests), ref, rtol, atol)
    drives.compare(drives.drive_prefill_then_decode(runner(roomy, graph_max_len=192), requests),
                   ref, rtol, atol)
    drives.compare(drives.drive_portions(runner(roomy), requests), ref, rtol, atol)
    drives.compare(drives.drive_mixed(runner(320 // page), requests), ref, rtol, atol)
