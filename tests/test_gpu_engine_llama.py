"""The Llama decode stack served by the same engine as every model: registry -> model runner ->
cache manager -> scheduler -> sampler.  No second implementation exists for a synthetic stack, so
the checks are the engine's invariants on it: a prompt whole, in portions, and token by token
gives the same logits (fp16 rounding); a mixed step (portions beside single tokens, in any order)
equals each request alone; generation runs through the scheduler with a small token budget and
gives back every block."""
import json

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make(tmp_path):
    from vllm_legacy_amd.engine.cache_manager import CacheManager
    from vllm_legacy_amd.engine.llama_adapter import LlamaEngineConfig
    from vllm_legacy_amd.engine.model_runner import ModelRunner
    from vllm_legacy_amd.model.llama_decode import LlamaConfig
    from vllm_legacy_amd.model.registry import load_model
    cfg = LlamaEngineConfig(LlamaConfig.tiny(), quant="none", kv_cache_dtype="auto", seed=3)
    (tmp_path / "llama").mkdir()
    (tmp_path / "llama" / "config.json").write_text(json.dumps(cfg.to_dict()))
    model = load_model(str(tmp_path / "llama"), torch.float16, DEV)
    cache = CacheManager(64, 16, 4)
    return model, cache, ModelRunner(model, cache, DEV)


def run(runner, cache, done, entries):
    batch, want = [], []
    for sid, tokens in entries:
        if not cache.is_live(sid):
            cache.admit(sid)
            done[sid] = 0
        cache.grow(sid, done[sid] + len(tokens))
        batch.append((sid, list(tokens), done[sid]))
        want.append(list(range(len(tokens))))
    logits = runner.execute(batch, want).cpu()
    out, at = {}, 0
    for sid, tokens in entries:
        out[sid] = logits[at:at + len(tokens)]
        at += len(tokens)
        done[sid] += len(tokens)
    return out


def close(a, b):
    err = float((a - b).abs().max() / b.abs().max())
    assert err <= 2e-2, err


def test_portions_decoding_and_mixed_steps_agree(tmp_path):
    model, cache, runner = make(tmp_path)
    g = torch.Generator().manual_seed(0)
    a = torch.randint(0, 1024, (45, ), generator=g).tolist()
    b = torch.randint(0, 1024, (20, ), generator=g).tolist()
    done = {}
    whole_a = run(runner, cache, done, [("a", a)])["a"]
    whole_b = run(runner, cache, done, [("b", b)])["b"]
    cache.free("a")
    cache.free("b")
    done.clear()
    parts = [run(runner, cache, done, [("a", a[:17])])["a"], run(runner, cache, done, [("a", a[17:40])])["a"]]
    parts += [run(runner, cache, done, [("a", a[t:t + 1])])["a"] for t in range(40, 45)]
    close(torch.cat(parts), whole_a)
    cache.free("a")
    done.clear()
    # a mixed step in the engine's order: a single token before a portion
    run(runner, cache, done, [("b", b[:19])])
    first = run(runner, cache, done, [("b", b[19:]), ("a", a[:30])])
    second = run(runner, cache, done, [("a", a[30:])])
    close(first["b"], whole_b[19:])
    close(torch.cat([first["a"], second["a"]]), whole_a)


def test_generation_through_the_scheduler(tmp_path):
    from vllm_legacy_amd.engine import EngineConfig, LLMEngine, SamplingParams
    model, _, _ = make(tmp_path)
    engine = LLMEngine(model, EngineConfig(block_size=16, num_blocks=32, max_num_seqs=3, max_num_batched_tokens=24), DEV)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, 1024, (n, ), generator=g).tolist() for n in (40, 5, 1, 18)]
    outs = engine.generate(prompts, SamplingParams(max_tokens=6))
    assert [len(o.token_ids) for o in outs] == [6] * 4 and all(o.finished for o in outs)
    assert engine.cache.free_blocks == 32 and engine.cache.free_slots == 3
