"""bin/trace_run as a user runs it: a child process fed JSON steps, logits read back
from the files it writes.  The same requests are replayed whole, with the last 32
tokens one by one, in portions of changing size, and mixed with so few pages that they
are used again; every variant must give the plain implementation's logits, in float32
and in bfloat16."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from helpers import TINY, random_prompt
from plain import qwen3_plain as plain
from tokensprint_amd.weights import write_random_model

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
TOL = {"float32": (1e-4, 2e-5), "bfloat16": (3e-2, 3e-2)}


class TraceClient:
    def __init__(self, model_dir, dtype, out_dir, max_tokens, vocab):
        self.out_dir, self.vocab, self.n = Path(out_dir), vocab, 0
        self.proc = subprocess.Popen(
            [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir),
             "--dtype", dtype, "--out", str(out_dir), "--max-tokens", str(max_tokens)],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)

    def step(self, entries, end=()):
        """entries: [(id, tokens, want)].  Returns {id: {offset: logits row}}."""
        rec = {"step": self.n, "entries": [{"id": i, "tokens": t, "want": w}
                                           for i, t, w in entries], "end": list(end)}
        self.proc.stdin.write(json.dumps(rec) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline().strip()
        assert line == f"done {self.n}", f"trace_run said {line!r}"
        out = {}
        wanted = sum(len(w) for _, _, w in entries)
        if wanted:
            data = np.fromfile(self.out_dir / f"{self.n}.f32", dtype="<f4")
            data = data.reshape(wanted, self.vocab)
            row = 0
            for i, _, w in entries:
                for off in w:
                    out.setdefault(i, {})[off] = torch.from_numpy(data[row].copy())
                    row += 1
        else:
            assert not (self.out_dir / f"{self.n}.f32").exists()
        self.n += 1
        return out

    def close(self):
        self.proc.stdin.close()
        assert self.proc.wait(timeout=60) == 0


def check(got, ref, rtol, atol, what):
    for rid, rows in got.items():
        assert sorted(rows) == list(range(ref[rid].shape[0])), f"{what} {rid}: missing positions"
        g = torch.stack([rows[p] for p in sorted(rows)])
        bad = ~torch.isclose(g, ref[rid], rtol=rtol, atol=atol)
        assert not bad.any(), (f"{what}: request {rid}, first wrong position "
                               f"{int(bad.any(1).nonzero()[0])}, error {(g - ref[rid]).abs().max():.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_replay_variants(tmp_path, name, dtype):
    cfg, seed, _ = TINY[name]
    model_dir = write_random_model(tmp_path / "model", cfg, seed,
                                   torch.float32 if dtype == "float32" else torch.bfloat16)
    pcfg, w = plain.read_model_dir(model_dir)
    vocab = cfg["vocab_size"]
    requests = {f"r{i}": random_prompt(n, vocab, 50 + i) for i, n in enumerate([70, 45, 100, 33, 64])}
    ref = {rid: plain.forward_logits(pcfg, w, t) for rid, t in requests.items()}
    rtol, atol = TOL[dtype]
    # live requests hold at most 128 + 64 + 128 + 64 tokens (rounded up to 64 each)
    client = TraceClient(model_dir, dtype, tmp_path / "out", 384, vocab)
    try:
        # 1. whole
        got = {}
        for rid, toks in requests.items():
            res = client.step([(rid, toks, list(range(len(toks))))], end=[rid])
            got[rid] = res[rid]
        check(got, ref, rtol, atol, "whole")
        # 2. most in one step, the last 32 one by one (a step with nothing wanted first)
        got = {}
        for rid, toks in requests.items():
            head = max(len(toks) - 32, 4)
            client.step([(rid, toks[:2], [])])
            rows = dict((k + 2, v) for k, v in client.step(
                [(rid, toks[2:head], list(range(head - 2)))])[rid].items())
            rows.update({0: ref[rid][0], 1: ref[rid][1]})      # not asked for
            for p in range(head, len(toks)):
                rows[p] = client.step([(rid, [toks[p]], [0])],
                                      end=[rid] if p == len(toks) - 1 else [])[rid][0]
            got[rid] = rows
        check(got, ref, rtol, atol, "tail one by one")
        # 3. portions of changing size, down to two tokens
        got = {}
        sizes = [7, 2, 13, 3, 2, 29, 5, 2, 64, 11]
        for rid, toks in requests.items():
            pos, i, rows = 0, 0, {}
            while pos < len(toks):
                n = min(sizes[i % len(sizes)], len(toks) - pos)
                i += 1
                res = client.step([(rid, toks[pos:pos + n], list(range(n)))],
                                  end=[rid] if pos + n == len(toks) else [])
                rows.update({pos + k: v for k, v in res[rid].items()})
                pos += n
            got[rid] = rows
        check(got, ref, rtol, atol, "portions")
        # 4. mixed: up to four live, portions beside single tokens, requests left out of
        #    steps, pages used again as requests end
        g = torch.Generator().manual_seed(1)
        got = {rid: {} for rid in requests}
        waiting, live = list(requests), {}
        while waiting or live:
            while waiting and len(live) < 4:
                live[waiting.pop(0)] = 0
            entries, ended = [], []
            for rid in list(live):
                if len(live) > 1 and float(torch.rand(1, generator=g)) < 0.2:
                    continue
                pos, toks = live[rid], requests[rid]
                left = len(toks) - pos
                n = 1 if left <= 10 else min(int(torch.randint(2, 20, (1,), generator=g)), left - 10)
                entries.append((rid, toks[pos:pos + n], list(range(n))))
                live[rid] = pos + n
                if pos + n == len(toks):
                    ended.append(rid)
            if not entries:
                continue
            res = client.step(entries, end=ended)
            for rid, toks, _ in entries:
                start = live[rid] - len(toks)
                got[rid].update({start + k: v for k, v in res[rid].items()})
            for rid in ended:
                del live[rid]
        check(got, ref, rtol, atol, "mixed")
    finally:
        client.close()
