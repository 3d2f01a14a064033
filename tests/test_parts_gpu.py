"""Each part alone against the plain functions, and toy parts registered from here:
a mixer with fixed-size state of its own, a feed-forward with routing, another position
encoding, a run order that names a layer twice and a layer that reads another run's
cache.  Nothing in the framework's files knows these parts."""

import pytest
import torch

from plain import qwen3_plain as plain
from tokensprint_amd.cache import CacheManager, CacheStorage
from tokensprint_amd.config.registry import _ARCHITECTURES, register_architecture
from tokensprint_amd.engine import ModelRunner, StepEntry
from tokensprint_amd.engine.assemble import random_model
from tokensprint_amd.engine.batch import BatchBuilder
from tokensprint_amd.models.spec import LayerSpec, ModelSpec, PartSpec, Run
from tokensprint_amd.parts import (EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, POSITIONS, Block,
                                   BuildContext, Embedding, FeedForward, Head, Mixer,
                                   PositionEncoding, SlotStateNeed, TensorDecl, build_part,
                                   register, NORMS, BLOCKS)

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def context(gpu_device, dtype, width):
    from tokensprint_amd.kernels import load_hip_ops
    return BuildContext(ops=load_hip_ops(gpu_device), dtype=dtype, device=gpu_device, width=width)


def one_request_batch(ctx, needs, tokens, page=8):
    storage = CacheStorage(needs, page, 32, 2, ctx.dtype, ctx.device)
    manager = CacheManager(storage.groups, page, 32, 2)
    rc = manager.admit("a")
    manager.extend(rc, tokens)
    batch = BatchBuilder(ctx.device, len(storage.groups)).build(
        [StepEntry(rc, [0] * tokens, 0, [tokens - 1])])
    return batch, storage


# ------------------------------------------------------------------ parts alone
@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(gpu_device, dtype):
    ctx = context(gpu_device, dtype, 96)
    norm = build_part(NORMS, PartSpec("rmsnorm", {"dim": 96, "eps": 1e-5, "weight": "w"}), ctx)
    w = 1 + 0.1 * rnd((96,), 1)
    norm.load({"w": w.to(gpu_device)}.get)
    x, d = rnd((9, 96), 2), rnd((9, 96), 3).to(dtype)
    ref = plain.rms_norm(x, w, 1e-5)
    torch.testing.assert_close(norm.forward(x.to(gpu_device)).float().cpu(), ref, **tol(dtype))
    resid = x.to(gpu_device)
    out = norm.add_forward(resid, d.to(gpu_device))
    torch.testing.assert_close(resid.cpu(), x + d.float())
    torch.testing.assert_close(out.float().cpu(), plain.rms_norm(x + d.float(), w, 1e-5), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotary_part(gpu_device, dtype):
    ctx = context(gpu_device, dtype, 64)
    rope = build_part(POSITIONS, PartSpec("rope", {"dim": 32, "theta": 1e6, "max_position": 300}), ctx)
    cos, sin = plain.rope_cos_sin(torch.arange(300), 32, 1e6)
    torch.testing.assert_close(rope.cos.cpu(), cos, rtol=0, atol=0)      # host-built table
    torch.testing.assert_close(rope.sin.cpu(), sin, rtol=0, atol=0)
    q = rnd((5, 4, 32), 4).to(dtype)
    pos = torch.tensor([0, 7, 299, 41, 2], dtype=torch.int32)
    ref = plain.apply_rope(q.float(), cos[pos.long()], sin[pos.long()])
    qd = q.to(gpu_device)
    rope.apply(qd, None, pos.to(gpu_device))
    torch.testing.assert_close(qd.float().cpu(), ref, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 5])
def test_attention_and_swiglu_and_block_parts(gpu_device, dtype, window):
    width, nq, nkv, hd, inner, T = 48, 6, 2, 16, 72, 21
    ctx = context(gpu_device, dtype, width)
    ctx.positions["rope"] = build_part(POSITIONS, PartSpec(
        "rope", {"dim": hd, "theta": 1e4, "max_position": 64}), ctx)
    layer = LayerSpec(
        block="pre_norm",
        mixer=PartSpec("gqa_attention", {"prefix": "a.", "num_heads": nq, "num_kv_heads": nkv,
                                         "head_dim": hd, "qk_norm": True, "qk_norm_eps": 1e-6,
                                         "position": "rope", "window": window}),
        feed_forward=PartSpec("swiglu", {"prefix": "f.", "inner_dim": inner}),
        mixer_norm=PartSpec("rmsnorm", {"dim": width, "eps": 1e-6, "weight": "n1"}),
        ffn_norm=PartSpec("rmsnorm", {"dim": width, "eps": 1e-6, "weight": "n2"}))
    mixer = build_part(MIXERS, layer.mixer, ctx)
    ffn = build_part(FEED_FORWARDS, layer.feed_forward, ctx)
    n1, n2 = build_part(NORMS, layer.mixer_norm, ctx), build_part(NORMS, layer.ffn_norm, ctx)
    w = {}
    for i, part in enumerate((mixer, ffn, n1, n2)):
        for name, decl in part.tensors().items():
            t = 1 + 0.1 * rnd(decl.shape, 10 + i) if decl.role == "vector" else rnd(decl.shape, 20 + i, 0.1)
            w[name] = t.to(dtype).float()              # the values the device holds
    dev = {k: v.to(gpu_device, torch.float32 if v.dim() == 1 else dtype) for k, v in w.items()}
    for part in (mixer, ffn, n1, n2):
        part.load(dev.get)
    batch, storage = one_request_batch(ctx, [mixer.cache_need()], T)
    h = rnd((T, width), 5).to(dtype)
    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, eps=1e-6, theta=1e4, window=window)
    pw = {"a." + k.split("a.", 1)[1]: v for k, v in w.items() if k.startswith("a.")}
    ref_attn = plain.attention_mixer(h.float(), pw, "a.", torch.arange(T), **kw)
    out = mixer.forward(h.to(gpu_device), batch, storage.views[0], True)
    torch.testing.assert_close(out.float().cpu(), ref_attn, **tol(dtype))
    ref_ffn = plain.swiglu(h.float(), w, "f.")
    torch.testing.assert_close(ffn.forward(h.to(gpu_device), batch).float().cpu(), ref_ffn, **tol(dtype))
    # the block: x + attn(norm(x)), then + ffn(norm(.))
    block = BLOCKS["pre_norm"]({"mixer": mixer, "feed_forward": ffn, "mixer_norm": n1,
                                "ffn_norm": n2}, ctx)
    x = rnd((T, width), 6)
    resid, delta = block.forward(x.to(gpu_device), None, batch, storage.views[0], True)
    x1 = x + plain.attention_mixer(plain.rms_norm(x, w["n1"], 1e-6).to(dtype).float(), pw, "a.",
                                   torch.arange(T), **kw)
    x2 = x1 + plain.swiglu(plain.rms_norm(x1, w["n2"], 1e-6).to(dtype).float(), w, "f.")
    torch.testing.assert_close((resid + delta.float()).cpu(), x2, **tol(dtype))


# ------------------------------------------------------------------ toy parts
class ToyDecayMixer(Mixer):
    """State s (one vector per request): s <- decay * s + x_t; output W s.  Tokens of a
    request must be taken in order, and the state lives in the request's slot between
    steps.  Written with torch operations: it stands for a part someone brings along.
    It reads the slot ids back to the host, so it cannot run inside a captured graph and
    says so."""

    capturable = False

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.name, self.decay = params["weight"], params["decay"]

    def tensors(self):
        return {self.name: TensorDecl((self.ctx.width, self.ctx.width))}

    def load(self, get):
        self.w = get(self.name)

    def cache_need(self):
        return SlotStateNeed((self.ctx.width,), torch.float32)

    def forward(self, h, batch, cache, write_cache):
        out = torch.empty_like(h)
        first = 0
        slots = batch.slot_ids.tolist()
        for b, n in enumerate(batch.q_lens):
            s = cache.state[slots[b]]
            if batch.starts[b] == 0:
                s.zero_()
            for t in range(first, first + n):
                s.mul_(self.decay).add_(h[t].float())
                out[t] = (self.w.float() @ s).to(h.dtype)
            first += n
        return out


class ToyDecayMixerOnDevice(ToyDecayMixer):
    """The same mixer with a decode step (one token per entry) that touches device tensors
    only, so it may be captured: the state rows of the step's slots are gathered, updated
    and scattered back.  Idle lanes of a captured batch carry the slot no request owns."""

    capturable = True

    def forward(self, h, batch, cache, write_cache):
        if batch.max_q_len > 1:
            return super().forward(h, batch, cache, write_cache)
        slots = batch.slot_ids.long()
        s = cache.state.index_select(0, slots)
        s = torch.where((batch.positions == 0)[:, None], torch.zeros_like(s), s)
        s = s * self.decay + h.float()
        cache.state.index_copy_(0, slots, s)
        return (s @ self.w.float().T).to(h.dtype)


class ToyTop1FeedForward(FeedForward):
    """Two experts, each one matrix; a router picks one per token (float32 logits)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.prefix = params["prefix"]

    def tensors(self):
        W = self.ctx.width
        return {self.prefix + "router": TensorDecl((2, W)),
                self.prefix + "e0": TensorDecl((W, W)), self.prefix + "e1": TensorDecl((W, W))}

    def load(self, get):
        self.router, self.e = get(self.prefix + "router"), [get(self.prefix + "e0"), get(self.prefix + "e1")]

    def forward(self, h, batch):
        pick = (h.float() @ self.router.float().T).argmax(-1)
        if batch.max_q_len == 1:
            # a decode step may be captured: no row lists on the host, both experts run
            # and each token keeps its own
            both = [self.ops.linear(h, e, h.dtype) for e in self.e]
            return torch.where((pick == 0)[:, None], both[0], both[1])
        out = torch.zeros_like(h)
        for i in (0, 1):
            rows = (pick == i).nonzero().squeeze(-1)
            if rows.numel():
                out[rows] = self.ops.linear(h[rows].contiguous(), self.e[i], h.dtype)
        return out


class ToyOffsetEncoding(PositionEncoding):
    """Adds position * step to every query and key element: no rotary table, so the
    attention part takes its unfused path (norm, this encoding, store)."""

    def apply(self, q, k, positions):
        shift = (positions.float() * self.params["step"])[:, None, None]
        q.copy_((q.float() + shift).to(q.dtype))
        if k is not None:
            k.copy_((k.float() + shift).to(k.dtype))


class ToyScaledEmbedding(Embedding):
    """Rows of the table times a constant (as architectures that scale their embeddings by
    the root of the width do)."""

    def forward(self, token_ids):
        return super().forward(token_ids) * self.params["scale"]


class ToyCappedHead(Head):
    """Logits squashed into (-cap, cap): cap * tanh(logits / cap)."""

    def forward_from_stream(self, resid, delta, norm):
        cap = self.params["cap"]
        return cap * torch.tanh(super().forward_from_stream(resid, delta, norm) / cap)


class ToySandwichBlock(Block):
    """A layer without a feed-forward whose mixer sits between two norms:
    x = x + post_norm(mixer(mixer_norm(x)))."""

    ROLES = {"mixer_norm": (NORMS, True), "mixer": (MIXERS, True), "post_norm": (NORMS, True)}

    def forward(self, resid, delta, batch, cache, write_cache, next_hint=None):
        h = self.mixer_norm.forward(resid) if delta is None \
            else self.mixer_norm.add_forward(resid, delta)
        return resid, self.post_norm.forward(self.mixer.forward(h, batch, cache, write_cache))


def toy_spec(raw):
    W, V = raw["width"], raw["vocab"]
    norm = lambda name: PartSpec("rmsnorm", {"dim": W, "eps": 1e-5, "weight": name})
    attn = lambda prefix, pos, own=True: PartSpec("gqa_attention", {
        "prefix": prefix, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16, "qk_norm": own,
        "qk_norm_eps": 1e-5, "position": pos, "own_kv": own})
    layers = (
        LayerSpec("pre_norm", attn("l0.attn.", "offset"), PartSpec("swiglu", {"prefix": "l0.ffn.", "inner_dim": 40}),
                  norm("l0.n1"), norm("l0.n2")),
        LayerSpec("pre_norm", PartSpec(raw.get("decay_mixer", "toy_decay"),
                                       {"weight": "l1.mix", "decay": 0.5}),
                  PartSpec("toy_top1", {"prefix": "l1.ffn."}), norm("l1.n1"), norm("l1.n2")),
        LayerSpec("pre_norm", attn("l2.attn.", "rope", own=False), PartSpec("swiglu", {"prefix": "l2.ffn.", "inner_dim": 24}),
                  norm("l2.n1"), norm("l2.n2")),
        # a block kind of the test's own: no feed-forward, a norm behind the mixer
        LayerSpec("toy_sandwich", mixer=attn("l3.attn.", "rope"), mixer_norm=norm("l3.n1"),
                  post_norm=norm("l3.post")),
        # and a pre-norm layer that is a feed-forward only: its run owns no cache
        LayerSpec("pre_norm", feed_forward=PartSpec("swiglu", {"prefix": "l4.ffn.", "inner_dim": 56}),
                  ffn_norm=norm("l4.n2")),
    )
    return ModelSpec(
        architecture="ToyForTests", width=W, vocab_size=V,
        embedding=PartSpec("toy_scaled_embedding", {"weight": "embed", "vocab_size": V, "scale": 3.0}),
        positions={"offset": PartSpec("toy_offset", {"step": 0.01}),
                   "rope": PartSpec("rope", {"dim": 16, "theta": 100.0, "max_position": 128})},
        layers=layers,
        # layer 0 runs twice (two caches of its own); layer 2 reads the cache of run 0
        order=(Run(0), Run(1), Run(0), Run(2, cache_of=0), Run(3), Run(4)),
        final_norm=norm("final"),
        head=PartSpec("toy_capped_head", {"weight": "embed", "vocab_size": V, "tied": True, "cap": 2.0}),
        max_position=128)


@pytest.fixture(scope="module")
def toy_registered():
    for reg, kind, cls in ((MIXERS, "toy_decay", ToyDecayMixer),
                           (MIXERS, "toy_decay_on_device", ToyDecayMixerOnDevice),
                           (FEED_FORWARDS, "toy_top1", ToyTop1FeedForward),
                           (POSITIONS, "toy_offset", ToyOffsetEncoding),
                           (EMBEDDINGS, "toy_scaled_embedding", ToyScaledEmbedding),
                           (HEADS, "toy_capped_head", ToyCappedHead),
                           (BLOCKS, "toy_sandwich", ToySandwichBlock)):
        register(reg, kind, replace=True)(cls)
    if "ToyForTests" not in _ARCHITECTURES:
        register_architecture("ToyForTests", parse_config=lambda raw: raw, build_spec=toy_spec)
    return {"architectures": ["ToyForTests"], "width": 64, "vocab": 97}


def toy_plain(model, tokens):
    """The toy model on a whole sequence, without caches, from the plain functions."""
    g = lambda t: t.float().cpu()
    b = model.blocks
    T = len(tokens)
    pos = torch.arange(T)
    x = 3.0 * g(model.embedding.table)[tokens]

    def attention(blk, h, k_src, mode):
        m = blk.mixer
        qkv = h @ g(m.w_qkv).T
        q = plain.rms_norm(qkv[:, :64].view(T, 4, 16), g(m.w_qnorm), 1e-5) if m.w_qnorm is not None \
            else qkv[:, :64].view(T, 4, 16)
        if mode == "offset":
            k = plain.rms_norm(qkv[:, 64:96].view(T, 2, 16), g(m.w_knorm), 1e-5)
            v = qkv[:, 96:].view(T, 2, 16)
            shift = (pos.float() * 0.01)[:, None, None]
            q, k = q + shift, k + shift
        else:
            cos, sin = plain.rope_cos_sin(pos, 16, 100.0)
            q = plain.apply_rope(q, cos, sin)
            if k_src is None:          # a layer with keys of its own behind the rotation
                k = plain.apply_rope(plain.rms_norm(qkv[:, 64:96].view(T, 2, 16), g(m.w_knorm), 1e-5),
                                     cos, sin)
                v = qkv[:, 96:].view(T, 2, 16)
            else:
                k, v = k_src
        o = plain.causal_attention(q, k, v)
        return o.reshape(T, 64) @ g(m.w_o).T, (k, v)

    def swiglu(blk, h):
        f = blk.feed_forward
        gu = h @ g(f.w_gate_up).T
        i = gu.shape[1] // 2
        return (torch.nn.functional.silu(gu[:, :i]) * gu[:, i:]) @ g(f.w_down).T

    norm = lambda n, t: plain.rms_norm(t, g(n.weight), 1e-5)
    a, kv0 = attention(b[0], norm(b[0].mixer_norm, x), None, "offset")          # run 0
    x = x + a
    x = x + swiglu(b[0], norm(b[0].ffn_norm, x))
    h = norm(b[1].mixer_norm, x)                                                 # run 1
    s, outs = torch.zeros(64), []
    for t in range(T):
        s = 0.5 * s + h[t]
        outs.append(g(b[1].mixer.w) @ s)
    x = x + torch.stack(outs)
    h = norm(b[1].ffn_norm, x)
    pick = (h @ g(b[1].feed_forward.router).T).argmax(-1)
    e = [g(w) for w in b[1].feed_forward.e]
    x = x + torch.stack([e[int(p)] @ h[t] for t, p in enumerate(pick)])
    a, _ = attention(b[0], norm(b[0].mixer_norm, x), None, "offset")             # run 2: layer 0 again
    x = x + a
    x = x + swiglu(b[0], norm(b[0].ffn_norm, x))
    a, _ = attention(b[2], norm(b[2].mixer_norm, x), kv0, "rope")                # run 3 reads run 0's cache
    x = x + a
    x = x + swiglu(b[2], norm(b[2].ffn_norm, x))
    a, _ = attention(b[3], norm(b[3].mixer_norm, x), None, "rope")               # run 4: the sandwich
    x = x + norm(b[3].post_norm, a)
    assert b[3].parts() == [b[3].mixer_norm, b[3].mixer, b[3].post_norm] and b[4].mixer is None
    x = x + swiglu(b[4], norm(b[4].ffn_norm, x))                                 # run 5: feed-forward only
    return 2.0 * torch.tanh(norm(model.final_norm, x) @ g(model.embedding.table).T / 2.0)


def test_toy_parts_build_and_step(toy_registered, gpu_device):
    _, model = random_model(toy_registered, seed=5, dtype=torch.float32, device=gpu_device, std=0.2)
    needs = model.cache_needs()
    assert [type(n).__name__ for n in needs] == ["PagedKVNeed", "SlotStateNeed", "PagedKVNeed", "NoneType",
                                                 "PagedKVNeed", "NoneType"]
    runner = ModelRunner(model, page_size=4, num_pages=40, num_slots=3)
    assert len(runner.storage.groups) == 1 and runner.storage.groups[0].runs == (0, 2, 4)
    assert runner.storage.views[1].state.shape == (3 + 1, 64)     # one row for idle lanes
    g = torch.Generator().manual_seed(0)
    reqs = {rid: torch.randint(0, 97, (n,), generator=g).tolist() for rid, n in (("a", 30), ("b", 19), ("c", 44))}
    ref = {rid: toy_plain(model, toks) for rid, toks in reqs.items()}
    # mixed stepping: portions of changing size, three requests interleaved, slots reused
    got = {rid: {} for rid in reqs}
    live = {rid: [runner.manager.admit(rid), 0] for rid in ("a", "b")}
    sizes = [5, 1, 2, 9, 1, 3, 7, 1]
    step = 0
    while live:
        entries = []
        for rid, (rc, pos) in list(live.items()):
            n = min(sizes[(step + len(rid) + pos) % len(sizes)], len(reqs[rid]) - pos)
            runner.manager.extend(rc, pos + n)
            entries.append(StepEntry(rc, reqs[rid][pos:pos + n], pos, list(range(n))))
            live[rid][1] = pos + n
        logits = runner.step(entries).cpu()
        row = 0
        for e in entries:
            for wnt in e.want:
                got[e.cache.request_id][e.start + wnt] = logits[row]
                row += 1
        for rid in [r for r, (rc, pos) in live.items() if pos == len(reqs[r])]:
            runner.manager.free(live.pop(rid)[0])
            if rid == "a":                       # "c" takes the slot "a" gave back
                live["c"] = [runner.manager.admit("c"), 0]
                assert live["c"][0].slot == 0
        step += 1
    for rid in reqs:
        out = torch.stack([got[rid][p] for p in range(len(reqs[rid]))])
        torch.testing.assert_close(out, ref[rid], rtol=2e-4, atol=2e-4)


def toy_greedy(model, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(toy_plain(model, tokens)[-1].argmax()))
    return tokens[len(prompt):]


@pytest.mark.parametrize("mixer", ["toy_decay", "toy_decay_on_device"])
def test_toy_architecture_generates_through_the_engine(toy_registered, gpu_device, tmp_path, mixer):
    """The toy architecture behind LLMEngine.generate: scheduler, portions, a pool so small
    that requests are preempted and recomputed, and captured decode steps.  The mixer
    that reads its slots back to the host keeps every step eager by declaring itself not
    capturable; its device-only twin is captured, idle lanes included."""
    from tokensprint_amd.config import Config, SamplingParams
    from tokensprint_amd.engine.llm_engine import LLMEngine
    raw = dict(toy_registered, decay_mixer=mixer)
    _, model = random_model(raw, seed=5, dtype=torch.float32, device=gpu_device, std=0.2)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, 97, (n,), generator=g).tolist() for n in (9, 1, 30, 17, 22)]
    want = [toy_greedy(model, p, 10) for p in prompts]
    sp = SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)
    for pages in (64, 14):
        engine = LLMEngine(model, Config(
            model=str(tmp_path), max_model_len=128, dtype=torch.float32, kvcache_block_size=4,
            num_kvcache_blocks=pages, max_num_seqs=3, max_num_batched_tokens=16,
            chunked_prefill=True))
        captured = mixer == "toy_decay_on_device"
        assert bool(engine.runner.buckets) == captured
        assert set(engine.runner.graphs) == ({1, 2, 3} if captured else set())
        assert engine.generate(prompts, sp, use_tqdm=False) == want, pages
        if pages == 14:
            assert engine.scheduler.num_preemptions > 0
        engine.runner.manager.check()
    with pytest.raises(ValueError, match="fixed-size state"):
        LLMEngine(model, Config(model=str(tmp_path), max_model_len=128, dtype=torch.float32,
                                kvcache_block_size=4, num_kvcache_blocks=32, max_num_seqs=3,
                                enable_prefix_caching=True))
