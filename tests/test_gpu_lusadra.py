"""Lusadra through the framework -- registry, checkpoint loader, cache manager, model runner,
scheduler, sampler -- against the float64 reference of tests/lusadra_oracle.py on small random
models written to a temporary checkpoint folder.

Covered: whole prompts; prefill against token-by-token decoding; portions of several sizes down to
two tokens; batches of unequal requests against each alone; pages and state slots that are freed
and used again; windows that pass over page borders in prompts and in decoding; the first tokens;
long decoding; several size combinations (per-layer sizes, kv heads = heads, one head, a window of
one, no feed-forward, loops that start late / run once / run three times, odd sizes); float32 and
bfloat16; greedy generation through LLMEngine.generate, with and without preemption; the trace
replayer as a program.  The float32 bar is float32 rounding through the stack (1e-4 of the logits'
spread) and is the one that finds faults of cutting, batching and reuse: both number formats run the
same code.  The bfloat16 runs check that path's kernels; widths of 64 average little rounding noise
out, so their bar is loose (every position within 0.2 of the logits' spread, 0.05 on average)."""
import json
import os
import subprocess
import sys

import pytest
import torch

from tests import lusadra_oracle as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BAR = {torch.float32: 1e-4, torch.bfloat16: 0.2}
MEAN_BAR = {torch.float32: 1e-4, torch.bfloat16: 0.05}

CONFIGS = {
    "plain": dict(),
    "loop3": dict(layers=3, loop=(1, 3, 3), per_layer=[{}, {"heads": 6, "kv_heads": 3, "dim": 24, "window": 9, "ff": None},
                                                        {"r_heads": 3, "r_dim": 12, "r_vdim": 20, "tau": 7.0, "window": 3}]),
    "once": dict(layers=2, loop=(0, 2, 1), heads=4, kv_heads=4, window=1, r_heads=1, r_dim=16, r_vdim=8, ff=100),
    "odd": dict(width=96, layers=2, loop=(0, 1, 2), heads=3, kv_heads=1, dim=40, window=21, r_heads=2, r_dim=5,
                r_vdim=70, ff=130, temp_every=5, vocab=131),
    # head sizes the matrix-core prompt kernel takes (multiples of 32) with more query heads per KV
    # head than one workgroup holds
    "mfma": dict(width=128, layers=2, loop=(0, 2, 2), heads=10, kv_heads=2, dim=32, window=37, r_heads=2, r_dim=16,
                 r_vdim=32, ff=64, per_layer=[{}, {"heads": 2, "kv_heads": 1, "dim": 64, "window": 8}]),
    "wide_window": dict(layers=1, heads=2, kv_heads=2, dim=16, window=70, temp_every=64, loop=(0, 1, 2)),
}


class Served:
    """A checkpoint on disk, loaded through the registry, with the engine's cache manager and
    model runner around it."""

    def __init__(self, tmp_path, name, dtype, num_blocks=64, block_size=4, num_slots=3, seed=0):
        from vllm_legacy_amd.engine.cache_manager import CacheManager
        from vllm_legacy_amd.engine.model_runner import ModelRunner
        from vllm_legacy_amd.model.registry import load_model
        self.cfg = R.make_config(**CONFIGS[name])
        self.W = R.make_weights(self.cfg, seed=seed)
        self.folder = R.write_checkpoint(str(tmp_path / name), self.cfg, self.W)
        self.dtype = dtype
        self.model = load_model(self.folder, dtype, DEV)
        self.cache = CacheManager(num_blocks, block_size, num_slots)
        self.runner = ModelRunner(self.model, self.cache, DEV)
        self.done = {}

    def step(self, entries):
        """entries: [(id, tokens)]; logits of every token come back per id."""
        batch, want = [], []
        for sid, tokens in entries:
            if not self.cache.is_live(sid):
                self.cache.admit(sid)
                self.done[sid] = 0
            self.cache.grow(sid, self.done[sid] + len(tokens))
            batch.append((sid, list(tokens), self.done[sid]))
            want.append(list(range(len(tokens))))
        logits = self.runner.execute(batch, want).cpu()
        out, at = {}, 0
        for sid, tokens in entries:
            out[sid] = logits[at:at + len(tokens)]
            at += len(tokens)
            self.done[sid] += len(tokens)
        return out

    def end(self, sid):
        self.cache.free(sid)
        del self.done[sid]

    def reference(self, tokens):
        return R.model_forward(self.cfg, self.W, tokens)

    def check(self, got, tokens, what=""):
        within(R.logit_error(got, self.reference(tokens)), self.dtype, what)


def within(err, dtype, what=""):
    assert float(err.max()) <= BAR[dtype] and float(err.mean()) <= MEAN_BAR[dtype], (what, float(err.max()), float(err.mean()))


def tokens_of(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n, ), generator=g).tolist()


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt_portions_and_decoding_agree_with_the_reference(tmp_path, name, dtype):
    s = Served(tmp_path, name, dtype)
    n = 90 if name in ("wide_window", "mfma") else 41
    toks = tokens_of(s.cfg, n, 1)
    want = s.reference(toks)

    def run(sizes, sid):
        got, lo, i = [], 0, 0
        while lo < n:
            c = min(sizes[i % len(sizes)], n - lo)
            got.append(s.step([(sid, toks[lo:lo + c])])[sid])
            lo += c
            i += 1
        s.end(sid)
        return torch.cat(got)

    for sid, sizes in (("whole", [n]), ("portions", [2, 3, 4, 5, 1, 7, 2]), ("prefill+decode", [n - 12] + [1] * 12),
                       ("long portions", [33, 40, 5]), ("tokens", [1])):
        within(R.logit_error(run(sizes, sid), want), dtype, sid)


def test_layer_by_layer_against_the_reference(tmp_path):
    """The residual stream after every layer run, float32."""
    from vllm_legacy_amd.attention.batch import SequenceBatch
    s = Served(tmp_path, "loop3", torch.float32)
    toks = tokens_of(s.cfg, 17, 4)
    taps = []
    R.model_forward(s.cfg, s.W, toks, taps)
    s.cache.admit("a")
    s.cache.grow("a", 17)
    batch = SequenceBatch.build([17], [0], [s.cache.block_table("a")], [s.cache.state_slot("a")], 4, DEV)
    got = []
    with torch.inference_mode():
        s.model(torch.tensor(toks, device=DEV), batch.positions, s.runner.caches, batch,
                tap=lambda run, x: got.append(x.detach().cpu().clone()))
    assert len(got) == len(taps) == 1 + 2 * 3
    for run, (a, b) in enumerate(zip(got, taps)):
        assert float((a.to(R.F) - b).abs().max() / b.abs().max()) <= 2e-5, run


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixed_batches_with_pages_and_slots_used_again(tmp_path, dtype):
    """Three slots, a pool that cannot hold all five requests at once: requests end, their
    pages and slots go to later ones; every step mixes portions and single tokens."""
    s = Served(tmp_path, "loop3", dtype, num_blocks=30, block_size=4, num_slots=3)
    reqs = {k: tokens_of(s.cfg, n, i) for i, (k, n) in enumerate([("a", 45), ("b", 9), ("c", 30), ("d", 38), ("e", 2)])}
    plan = [
        [("a", 5), ("b", 2)],
        [("a", 16), ("b", 1), ("c", 2)],
        [("b", 1), ("c", 7), ("a", 1)],
        [("a", 9), ("b", 5), ("c", 1)],          # b ends here (9 tokens)
        [("d", 3), ("a", 1), ("c", 13)],         # d takes b's slot and pages
        [("d", 1), ("a", 13), ("c", 7)],         # a and c end
        [("d", 30), ("e", 1)],
        [("e", 1), ("d", 1)],
        [("d", 3)],
    ]
    got = {k: [] for k in reqs}
    at = {k: 0 for k in reqs}
    used_slots = {}
    for step in plan:
        entries = [(k, reqs[k][at[k]:at[k] + n]) for k, n in step]
        out = s.step(entries)
        for k, n in step:
            used_slots.setdefault(k, s.cache.state_slot(k))
            got[k].append(out[k])
            at[k] += n
            if at[k] == len(reqs[k]):
                s.end(k)
    assert at == {k: len(v) for k, v in reqs.items()}
    assert used_slots["d"] == used_slots["b"] and len(set(used_slots.values())) == 3
    for k in reqs:
        s.check(torch.cat(got[k]), reqs[k], k)


def test_long_decoding_over_many_windows_and_pages(tmp_path):
    s = Served(tmp_path, "plain", torch.float32, num_blocks=80, block_size=4)
    toks = tokens_of(s.cfg, 230, 8)
    got = [s.step([("a", toks[:6])])["a"]]
    for t in range(6, 230):
        got.append(s.step([("a", toks[t:t + 1])])["a"])
    s.check(torch.cat(got), toks)


def test_long_prompts_walk_the_recurrence_in_pieces(tmp_path, monkeypatch):
    """Prompts long enough for the recurrent layer to cut them into pieces (cut short here so the
    reference stays quick), whole and in large portions beside a decoding request, against the
    reference; then decoding goes on from the state the pieces left."""
    from vllm_legacy_amd.attention.recurrent import GatedLinearRecurrence
    monkeypatch.setattr(GatedLinearRecurrence, "PIECE_ROWS", 16)
    s = Served(tmp_path, "loop3", torch.float32, num_blocks=80)
    a, b = tokens_of(s.cfg, 75, 5), tokens_of(s.cfg, 110, 6)
    got_a = [s.step([("a", a[:70])])["a"]] + [s.step([("a", a[t:t + 1])])["a"] for t in range(70, 75)]
    s.check(torch.cat(got_a), a, "whole + decode")
    s.end("a")
    got_b = [s.step([("b", b[:45])])["b"], s.step([("b", b[45:104]), ("a", a[:3])])["b"]]
    got_b += [s.step([("b", b[t:t + 1])])["b"] for t in range(104, 110)]
    s.check(torch.cat(got_b), b, "portions + decode")


def test_a_batch_does_not_change_a_request(tmp_path):
    """The same request alone and beside two others: equal beyond rounding (float32)."""
    s = Served(tmp_path, "odd", torch.float32)
    a, b, c = (tokens_of(s.cfg, n, i) for i, n in enumerate((33, 12, 50)))
    alone = torch.cat([s.step([("a", a[:20])])["a"], s.step([("a", a[20:])])["a"]])
    s.end("a")
    s.step([("c", c[:41])])
    first = s.step([("b", b[:5]), ("a", a[:20]), ("c", c[41:42])])["a"]
    second = s.step([("c", c[42:43]), ("a", a[20:]), ("b", b[5:])])["a"]
    both = torch.cat([first, second])
    assert float(R.logit_error(both, alone).max()) <= 1e-5


def greedy_reference(s, prompt, n):
    """(tokens, how clear each choice was): a choice closer than the bar is a tie."""
    toks, margins = list(prompt), []
    for _ in range(n):
        last = s.reference(toks)[-1]
        top = torch.topk(last, 2).values
        margins.append(float(top[0] - top[1]))
        toks.append(int(torch.argmax(last)))
    return toks[len(prompt):], margins


@pytest.mark.parametrize("num_blocks,preempt", [(64, False), (9, True)])
def test_greedy_generation_through_the_engine(tmp_path, num_blocks, preempt):
    from vllm_legacy_amd.engine import EngineConfig, LLMEngine, SamplingParams
    s = Served(tmp_path, "plain", torch.float32)
    engine = LLMEngine(s.model, EngineConfig(block_size=4, num_blocks=num_blocks, max_num_seqs=3,
                                             max_num_batched_tokens=7), DEV)
    prompts = [tokens_of(s.cfg, n, 20 + n) for n in (11, 3, 6, 1)]
    outs = engine.generate(prompts, SamplingParams(max_tokens=8))
    assert (engine.scheduler.num_preemptions > 0) == preempt
    assert engine.cache.free_blocks == num_blocks and engine.cache.free_slots == 3
    for p, o in zip(prompts, outs):
        want, margins = greedy_reference(s, p, 8)
        assert o.finished and o.finish_reason == "length" and len(o.token_ids) == 8
        for t, (a, b, m) in enumerate(zip(o.token_ids, want, margins)):
            if m < 1e-3:
                break                      # a tie within rounding: what follows may differ
            assert a == b, (t, a, b)


def test_stop_token_and_seeded_sampling(tmp_path):
    from vllm_legacy_amd.engine import EngineConfig, LLMEngine, SamplingParams
    s = Served(tmp_path, "plain", torch.float32)
    engine = LLMEngine(s.model, EngineConfig(block_size=4, num_blocks=64, max_num_seqs=2), DEV)
    p = tokens_of(s.cfg, 7, 3)
    first = engine.generate([p], SamplingParams(max_tokens=6))[0].token_ids
    out = engine.generate([p], SamplingParams(max_tokens=6, stop_token_ids=[first[2]]))[0]
    assert out.finish_reason == "stop" and out.token_ids == first[:first.index(first[2]) + 1]
    sp = SamplingParams(max_tokens=6, temperature=1.5, top_k=20, top_p=0.9, seed=5)
    a = engine.generate([p, p], [sp, sp])
    assert a[0].token_ids == a[1].token_ids        # same seed, same request: same draw


def test_trace_replayer_as_a_program(tmp_path):
    """bin/trace_run fed three steps (two requests, a portion beside a single token, a request
    that ends and whose id comes back as a new request) writes the logits the reference gives."""
    s = Served(tmp_path, "once", torch.float32)
    a, b = tokens_of(s.cfg, 9, 1), tokens_of(s.cfg, 4, 2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[6:7], "want": []}, {"id": "b", "tokens": b[:3], "want": [2]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[3:], "want": [0]}, {"id": "a", "tokens": a[7:], "want": [1]}], "end": ["a", "b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": b, "want": [3]}], "end": ["a"]},
    ]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", s.folder, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(x) for x in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    import numpy as np
    ra, rb = s.reference(a), s.reference(b)
    V = s.cfg["vocab"]
    want = {0: ra[[0, 5]], 1: rb[[2]], 2: torch.stack([rb[3], ra[8]]), 3: rb[[3]]}
    for n, w in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, V))
        assert got.shape == w.shape and float(R.logit_error(got, w).max()) <= 1e-4, n
