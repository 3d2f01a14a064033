"""The engine with the HIP kernels on the GPU against the plain implementation: every
way of cutting requests into steps, in float32 and in bfloat16, for the tiny
configurations.  Tolerances are fixed by the arithmetic (float32: a few units of
rounding over the depth; bfloat16: activations rounded to 8 bits between kernels), not
fitted to results."""

import pytest
import torch

import drives
from helpers import GPU_ONLY, TINY, WINDOWED, random_prompt
from plain import qwen3_plain as plain
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

TOL = {torch.float32: (1e-4, 2e-5), torch.bfloat16: (3e-2, 3e-2)}


CONFIGS = {**TINY, **GPU_ONLY, **WINDOWED}


@pytest.fixture(scope="module", params=[(n, d) for n in sorted(CONFIGS)
                                        for d in (torch.float32, torch.bfloat16)],
                ids=lambda p: f"{p[0]}-{str(p[1]).split('.')[-1]}")
def setup(request, tmp_path_factory, gpu_device):
    name, dtype = request.param
    cfg, seed, page = CONFIGS[name]
    d = tmp_path_factory.mktemp(f"tiny{name}")
    # (the wide models' values are drawn on the GPU, which takes a second where the CPU
    # takes a minute)
    write_random_model(d, cfg, seed, dtype, device="cpu" if name in TINY else gpu_device)
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


def test_preempted_and_recomputed(setup):
    """Requests that give everything back mid-way and are computed again from their first
    token beside the others' portions and decoded tokens (what the scheduler does when
    pages run out, engine/generation/scheduler.py:95-108,177-180 of the reference): the
    logits of both passes."""
    model, page, requests, ref, (rtol, atol) = setup
    runner = runner_for(model, page, 224 // page)
    drives.compare(drives.drive_preempted(runner, requests), ref, rtol, atol)
    assert all(pool.num_used == 0 for pool in runner.manager.pools)


def test_captured_decode_steps(setup):
    """Decode through captured graphs: every replay is checked against the plain logits,
    with eager steps (another request's prompt) between replays and two bucket sizes."""
    from tokensprint_amd.engine import StepEntry
    model, page, requests, ref, (rtol, atol) = setup
    runner = ModelRunner(model, page_size=page, num_pages=320 // page, num_slots=4,
                         graph_max_len=128)
    col = drives.Collector()
    ids = ["r3", "r4", "r7"]
    live = {}
    for rid in ids:
        rc = runner.manager.admit(rid)
        head = len(requests[rid]) - 30
        runner.manager.extend(rc, head)
        e = [StepEntry(rc, requests[rid][:head], 0, list(range(head)))]
        col.take(e, runner.step(e))
        live[rid] = [rc, head]
    for step in range(30):
        entries = []
        for rid in (ids if step % 3 else ids[:2]):          # buckets of 4 and of 2
            rc, pos = live[rid]
            if pos >= len(requests[rid]):
                continue
            runner.manager.extend(rc, pos + 1)
            entries.append(StepEntry(rc, requests[rid][pos:pos + 1], pos, [0]))
            live[rid][1] = pos + 1
        assert runner._graph_bucket(entries) in (2, 4)
        col.take(entries, runner.step(entries).clone())
        if step % 5 == 0:                                     # eager work between replays
            rc = runner.manager.admit("other")
            runner.manager.extend(rc, 17)
            runner.step([StepEntry(rc, requests["r2"], 0, [16])])
            runner.manager.free(rc)
    assert set(runner.graphs) == {2, 4}
    # finish the requests eagerly where steps were skipped
    for rid in ids:
        rc, pos = live[rid]
        while pos < len(requests[rid]):
            runner.manager.extend(rc, pos + 1)
            e = [StepEntry(rc, requests[rid][pos:pos + 1], pos, [0])]
            col.take(e, runner.step(e).clone())
            pos += 1
    drives.compare(col, {rid: ref[rid] for rid in ids}, rtol, atol)


def test_captured_decode_steps_with_many_requests(setup):
    """More than 16 requests decode together: the captured step then holds the vendor
    library's matrix products; replayed several times with eager steps between."""
    from tokensprint_amd.engine import StepEntry
    model, page, requests, ref, (rtol, atol) = setup
    runner = ModelRunner(model, page_size=page, num_pages=20 * (64 // page + 1), num_slots=20,
                         graph_max_len=64)
    toks = requests["r3"]                     # 40 tokens; 20 copies at staggered lengths
    col = drives.Collector()
    live = []
    for i in range(20):
        rc = runner.manager.admit(f"c{i}")
        head = 10 + i
        runner.manager.extend(rc, head)
        runner.step([StepEntry(rc, toks[:head], 0, [])])
        live.append([rc, head])
    for step in range(6):
        entries = []
        for rc, pos in live:
            runner.manager.extend(rc, pos + 1)
            entries.append(StepEntry(rc, toks[pos:pos + 1], pos, [0]))
        assert runner._graph_bucket(entries) == 20
        logits = runner.step(entries).clone()
        for (rc, pos), row in zip(live, logits):
            want = ref["r3"][pos]
            assert ((row.cpu() - want).abs() <= drives.row_tolerance(ref["r3"], rtol, atol)[pos]).all(), \
                f"step {step}, position {pos}: {(row.cpu() - want).abs().max():.3e}"
        for item in live:
            item[1] += 1
        if step % 2 == 0:                     # eager work between replays
            rc = live[0][0]
            runner.step([StepEntry(rc, toks[:3], 0, [2])])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_eps_of_the_per_head_norms_shows(name, dtype, tmp_path, gpu_device):
    """Random weights give head vectors far above eps, so a wrong eps in the q/k norm
    would pass every other test.  Here the q and k projections are scaled down until a
    head vector's mean square is near eps; the logits then depend on eps (the plain
    implementation with another eps is far outside the tolerance) and the engine must
    agree with the plain implementation at the configured one."""
    import json
    from safetensors.torch import save_file
    from tokensprint_amd.weights import random_tensors
    cfg, seed, page = TINY[name]
    cfg = dict(cfg, torch_dtype="float32" if dtype == torch.float32 else "bfloat16")
    tensors = random_tensors(cfg, seed, dtype=torch.float32)
    for key in tensors:
        if key.endswith(("q_proj.weight", "k_proj.weight")):
            tensors[key] = tensors[key] * 0.01
    tensors = {k: v.to(dtype).contiguous() for k, v in tensors.items()}
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file(tensors, str(tmp_path / "model.safetensors"))
    pcfg, w = plain.read_model_dir(tmp_path)
    _, model = load_model(tmp_path, dtype, gpu_device)
    requests = {"a": random_prompt(50, cfg["vocab_size"], 1), "b": random_prompt(37, cfg["vocab_size"], 2)}
    ref = {rid: plain.forward_logits(pcfg, w, t) for rid, t in requests.items()}
    rtol, atol = TOL[dtype]
    other = plain.forward_logits({**pcfg, "rms_norm_eps": pcfg["rms_norm_eps"] * 10}, w, requests["a"])
    # only the per-head norms can make this difference large: the block norms see the
    # same change in every other test's weights and move the logits far less.  In
    # float32 a wrong eps is 20 tolerances away; bfloat16's tolerance hides most of it
    margin = 20 if dtype == torch.float32 else 1.5
    assert (other - ref["a"]).abs().max() > margin * (atol + rtol * ref["a"].abs().max())
    col = drives.drive_prefill_then_decode(runner_for(model, page, 128 // page), requests, tail=12)
    drives.compare(col, ref, rtol, atol)


@pytest.fixture(scope="module", params=["E", "F"])
def wide_bfloat16(request, tmp_path_factory, gpu_device):
    cfg, seed, page = GPU_ONLY[request.param]
    d = tmp_path_factory.mktemp("wide" + request.param)
    write_random_model(d, cfg, seed, torch.bfloat16)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, torch.bfloat16, gpu_device)
    tokens = random_prompt(48, cfg["vocab_size"], 300)
    return model, page, tokens, plain.forward_logits(pcfg, w, tokens)


@pytest.mark.parametrize("captured", [False, True], ids=["eager", "captured"])
@pytest.mark.parametrize("lanes", [4, 5, 8, 9, 15, 16, 17, 32, 33, 64, 65, 127, 129])
def test_decode_lanes_on_both_sides_of_each_kernel_choice(wide_bfloat16, lanes, captured):
    """Which kernel serves a product depends on the number of rows: the output head goes
    to the library from 5 rows, the layer products of this width from 16, those with a
    short K from 17, everything from 65 (the 8B width, F); at the 0.6B width (E) the layer
    products are this engine's up to 64 rows, with more tiles of rows per workgroup from 17
    and from 33; and from 128 lanes (1,024 tiles of 16 query rows at 8 key/value heads) the
    step's attention is the kernel for long portions.  A decode step with one lane fewer and
    one lane more than each of these must give the plain logits, eagerly and from a captured
    graph."""
    from tokensprint_amd.engine import StepEntry
    model, page, tokens, ref = wide_bfloat16
    rtol, atol = TOL[torch.bfloat16]
    runner = ModelRunner(model, page_size=page, num_pages=lanes * (64 // page + 1),
                         num_slots=lanes, graph_max_len=64 if captured else None,
                         graph_max_batch=lanes)
    live = []
    for i in range(lanes):
        rc = runner.manager.admit(i)
        head = 8 + i % 30
        runner.manager.extend(rc, head)
        live.append([rc, head])
    # the prompts' heads, several requests a step
    for first in range(0, lanes, 16):
        runner.step([StepEntry(rc, tokens[:head], 0, []) for rc, head in live[first:first + 16]])
    for step in range(3):
        entries = []
        for rc, pos in live:
            runner.manager.extend(rc, pos + 1)
            entries.append(StepEntry(rc, tokens[pos:pos + 1], pos, [0]))
        assert (runner._graph_bucket(entries) is not None) == captured
        logits = runner.step(entries).float().cpu()
        bound = drives.row_tolerance(ref, rtol, atol)
        for (rc, pos), row in zip(live, logits):
            assert ((row - ref[pos]).abs() <= bound[pos]).all(), \
                f"{lanes} lanes, step {step}, position {pos}: {(row - ref[pos]).abs().max():.3e}"
        for item in live:
            item[1] += 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_long_prompt_through_the_kernels_of_many_rows(dtype, tmp_path, gpu_device):
    """A prompt of 777 tokens through a small model whose sizes (hidden 320, inner 768:
    multiples of 64 that are no powers of two) the LDS-tiled products take: whole (in
    bfloat16 the products carry the stream's add and the norm from 512 rows on, and the
    wide attention kernel takes the step), in portions of 477 and 300 (the separate
    kernels), and in a step of 601 rows that holds most of it beside a short prompt and
    another request's single token, all against the plain implementation."""
    from helpers import qwen3_config
    cfg = qwen3_config(hidden=320, layers=3, heads=4, kv_heads=2, head_dim=64, inter=768,
                       vocab=1000, eps=1e-6, theta=1e4, tied=True, max_pos=1024)
    write_random_model(tmp_path, cfg, 21, dtype, device=gpu_device)
    pcfg, w = plain.read_model_dir(tmp_path)
    _, model = load_model(tmp_path, dtype, gpu_device)
    requests = {"long": random_prompt(777, cfg["vocab_size"], 140)}
    ref = {rid: plain.forward_logits(pcfg, w, t) for rid, t in requests.items()}
    rtol, atol = TOL[dtype]
    runner = runner_for(model, 16, 777 // 16 + 2)
    ops, called = model.ctx.ops, []
    call = ops._call
    ops._call = lambda fn, *args: (called.append(fn.__name__), call(fn, *args))[1]
    try:
        drives.compare(drives.drive_whole(runner, requests), ref, rtol, atol)
        whole = list(called)
        drives.compare(drives.drive_portions(runner, requests, sizes=(477, 300)), ref, rtol, atol)
    finally:
        ops._call = call
    if dtype == torch.bfloat16:
        # every product that ends a sub-layer but the model's last, and every one behind
        # a norm but the first
        assert whole.count("ts_gemm_tiled_tail_bf16") == 2 * 3 - 1
        assert whole.count("ts_gemm_tiled_scaled_bf16") == 2 * 3 - 1
        assert "ts_gemm_tiled_tail_bf16" not in called[len(whole):]
    # and a step of as many rows made of three requests: most of the long prompt, a short
    # prompt whole and another request's single token
    from tokensprint_amd.engine import StepEntry
    more = {"a": random_prompt(40, cfg["vocab_size"], 141), "b": random_prompt(24, cfg["vocab_size"], 142)}
    ref.update({rid: plain.forward_logits(pcfg, w, t) for rid, t in more.items()})
    tokens = dict(requests, **more)
    runner = runner_for(model, 16, (777 + 40 + 24) // 16 + 4)
    rc = {rid: runner.manager.admit(rid) for rid in tokens}
    col = drives.Collector()

    def step(parts):
        entries = []
        for rid, lo, hi in parts:
            runner.manager.extend(rc[rid], hi)
            entries.append(StepEntry(rc[rid], tokens[rid][lo:hi], lo, list(range(hi - lo))))
        col.take(entries, runner.step(entries))

    step([("b", 0, 23)])
    step([("long", 0, 560), ("a", 0, 40), ("b", 23, 24)])
    step([("long", 560, 777)])
    for r in rc.values():
        runner.manager.free(r)
    runner.manager.check()
    drives.compare(col, ref, rtol, atol)
