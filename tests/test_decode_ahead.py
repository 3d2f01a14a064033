"""The engine's bookkeeping for decode steps launched ahead, on the CPU.

On the GPU a captured decode step leaves its drawn tokens on the device and the next
step may be launched before the host has read them.  Here the captured step is played by
a stand-in that runs the ordinary eager step of the torch kernel references and keeps the
last draw, so that what the engine does around it (which requests go on, whose lane is
dropped, pages taken ahead, admissions, preemption) is compared, token for token, with an
engine that never launches ahead.
"""

import pytest
import torch

from helpers import TINY, random_prompt
from kernel_refs import TorchOps
from tokensprint_amd.config import Config, SamplingParams
from tokensprint_amd.engine import StepEntry
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.engine.llm_engine import LLMEngine
from tokensprint_amd.weights import write_random_model


class _Passed:
    def synchronize(self):
        pass

    def record(self):
        pass


class CapturedStandIn:
    """`decode_and_sample` and `fits_captured` of a runner without graphs: greedy draws,
    tokens of lanes with a source taken from the draw before."""

    def __init__(self, runner):
        self.runner, self.last = runner, []
        self.calls = 0

    def fits_captured(self, entries):
        return all(len(e.tokens) == 1 and e.want == [0] for e in entries)

    def decode_and_sample(self, entries, temperatures, keys, sources=None):
        if not self.fits_captured(entries):
            return None
        assert all(t == 0.0 for t in temperatures)
        sources = sources or [-1] * len(entries)
        assert all(s < len(self.last) for s in sources)
        fed = [StepEntry(e.cache, [self.last[s]] if s >= 0 else e.tokens, e.start, [0])
               for e, s in zip(entries, sources)]
        logits = self.runner.step(fed)
        drawn = logits.argmax(dim=-1).to(torch.int32)
        self.last = drawn.tolist()
        self.calls += 1
        return drawn


def engine_for(model, d, ahead, **kw):
    args = dict(model=str(d), max_model_len=128, dtype=torch.float32, kvcache_block_size=16,
                num_kvcache_blocks=64, max_num_seqs=8, max_num_batched_tokens=48,
                chunked_prefill=True, decode_ahead=ahead)
    args.update(kw)
    engine = LLMEngine(model, Config(**args))
    stand_in = CapturedStandIn(engine.runner)
    engine.runner.decode_and_sample = stand_in.decode_and_sample
    engine.runner.fits_captured = stand_in.fits_captured
    engine._landing = [(torch.empty(64, dtype=torch.int32), _Passed()) for _ in range(2)]
    return engine


@pytest.fixture(scope="module", params=["A", "C"])
def setup(request, tmp_path_factory):
    cfg, seed, page = TINY[request.param]
    d = tmp_path_factory.mktemp(f"ahead{request.param}")
    write_random_model(d, cfg, seed, torch.float32)
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    prompts = [random_prompt(n, cfg["vocab_size"], 40 + i)
               for i, n in enumerate([5, 11, 17, 1, 23, 30, 8, 2, 13, 21])]
    return cfg, d, model, page, prompts


@pytest.mark.parametrize("kw", [dict(), dict(max_num_seqs=3), dict(pages_for=70),
                                dict(max_num_seqs=4, pages_for=100)],
                         ids=["roomy", "three-at-a-time", "tiny-pool", "both"])
def test_launching_ahead_changes_no_token(setup, kw):
    cfg, d, model, page, prompts = setup
    kw = dict(kw)
    if "pages_for" in kw:
        kw["num_kvcache_blocks"] = -(-kw.pop("pages_for") // page)
    L = min(cfg["max_position_embeddings"], 128)
    # an end-of-sequence token that greedy decoding does produce: taken from a first run
    probe = engine_for(model, d, False, kvcache_block_size=page, max_model_len=L)
    free_run = probe.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16,
                                                      ignore_eos=True), use_tqdm=False)
    eos = free_run[1][6]
    params = [SamplingParams(temperature=0.0, max_tokens=4 + 3 * i, ignore_eos=i % 3 == 0)
              for i in range(len(prompts))]
    outs = []
    for ahead in (False, True):
        engine = engine_for(model, d, ahead, kvcache_block_size=page, max_model_len=L, eos=eos,
                            **kw)
        outs.append(engine.generate(prompts, params, use_tqdm=False))
        engine.runner.manager.check()
        assert all(p.num_used == 0 for p in engine.runner.manager.pools)
        assert engine.is_finished()
        assert (engine.num_steps_ahead > 0) == ahead
        if "num_kvcache_blocks" in kw:
            assert engine.scheduler.num_preemptions > 0
    assert outs[0] == outs[1]
    stopped = [o for o, p in zip(outs[1], params) if not p.ignore_eos and eos in o]
    assert stopped and all(o.index(eos) == len(o) - 1 for o in stopped)


def test_a_step_ahead_is_not_launched_when_the_scheduler_has_to_decide(setup):
    cfg, d, model, page, prompts = setup
    L = min(cfg["max_position_embeddings"], 128)
    sp = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    engine = engine_for(model, d, True, kvcache_block_size=page, max_model_len=L, max_num_seqs=2)
    for p in prompts[:2]:
        engine.add_request(p, sp)
    engine.step()                       # both prompts in one step: not a captured step
    assert engine._flight is None
    engine.step()                       # first decode step; the second is launched with it
    assert engine._flight is not None and engine._flight.ahead
    # a newcomer while two run and two may: no room, the running ones go on ahead
    engine.add_request(prompts[2], sp)
    engine.step()
    assert engine._flight is not None
    # the last tokens of the two are known to be the last: nothing is launched past them,
    # and the newcomer starts in the step after
    while engine._flight is not None:
        engine.step()
    assert len(engine.scheduler.running) == 0 and len(engine.scheduler.waiting) == 1
    ahead_before = engine.num_steps_ahead
    engine.step()                       # the newcomer's prompt
    assert engine.num_steps_ahead == ahead_before
    while not engine.is_finished():
        engine.step()
    assert all(p.num_used == 0 for p in engine.runner.manager.pools)


def test_a_failure_around_a_step_ahead_leaves_the_engine_usable(setup):
    """A step launched ahead that fails (here: the runner raises) takes nothing with it:
    the pages it took go back, nothing stays in flight, and the engine finishes the same
    requests with the same tokens once the fault is gone."""
    cfg, d, model, page, prompts = setup
    L = min(cfg["max_position_embeddings"], 128)
    sp = SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True)
    want = engine_for(model, d, False, kvcache_block_size=page, max_model_len=L).generate(
        prompts[:3], sp, use_tqdm=False)
    engine = engine_for(model, d, True, kvcache_block_size=page, max_model_len=L)
    ordinals = [engine.add_request(p, sp) for p in prompts[:3]]
    engine.step()                       # the prompts
    engine.step()                       # a decode step, and one launched ahead of it
    assert engine._flight is not None and engine._flight.ahead
    good = engine.runner.decode_and_sample
    calls = {"n": 0}

    def failing(entries, temperatures, keys, sources=None):
        calls["n"] += 1
        raise RuntimeError("the device refused")

    engine.runner.decode_and_sample = failing
    with pytest.raises(RuntimeError, match="refused"):
        engine.step()                   # finishes the step in flight, fails launching ahead
    assert calls["n"] == 1 and engine._flight is None
    engine.runner.manager.check()
    for req in engine.scheduler.running:            # each holds its tokens' pages, no more
        assert len(req.cache.tables[0]) == -(-req.cache.num_tokens // page)
    engine.runner.decode_and_sample = good
    # the step that was in flight when the launch failed is lost with its tokens (its
    # requests are one token short and compute it again): same tokens in the end
    outputs = {}
    while not engine.is_finished():
        for ordinal, tokens in engine.step()[0]:
            outputs[ordinal] = tokens
    assert [outputs[o] for o in ordinals] == want
    assert all(p.num_used == 0 for p in engine.runner.manager.pools)
