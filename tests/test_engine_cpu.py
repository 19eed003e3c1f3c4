"""Host-side parts of the serving engine, no GPU: configuration reader, order of layer runs,
checkpoint reader, registry, cache manager (blocks and slots come back and are reused), step
metadata, scheduler policy (decodes first, prompts in portions, preemption), sampler."""
import json

import pytest
import torch

from tests import lusadra_oracle as R
from vllm_legacy_amd.attention.batch import SequenceBatch
from vllm_legacy_amd.engine.cache_manager import CacheManager
from vllm_legacy_amd.engine.sampling import Sampler, SamplingParams
from vllm_legacy_amd.engine.scheduler import Scheduler, Sequence
from vllm_legacy_amd.model import registry
from vllm_legacy_amd.model.lusadra import LusadraConfig
from vllm_legacy_amd.model_loader.safetensors_file import load_safetensors


def test_config_reader_takes_every_size_from_the_entry():
    cfg = R.make_config(layers=3, per_layer=[{}, {"heads": 6, "kv_heads": 3, "dim": 24, "window": 9, "ff": None},
                                             {"r_heads": 3, "r_dim": 12, "r_vdim": 20, "tau": 7.0}],
                        loop=(1, 3, 2))
    c = LusadraConfig.from_dict(json.loads(json.dumps(cfg)))
    assert (c.layers[1].left.heads, c.layers[1].left.kv_heads, c.layers[1].left.dim, c.layers[1].left.window) == (6, 3, 24, 9)
    assert c.layers[1].ff == 0 and c.layers[0].ff == 48
    assert (c.layers[2].right.heads, c.layers[2].right.dim, c.layers[2].right.vdim, c.layers[2].right.tau) == (3, 12, 20, 7.0)
    assert c.layers[0].left.temp_coef == 0.25 and c.layers[0].left.temp_every == 4
    assert c.layer_runs() == [(0, None), (1, 0), (2, None), (1, 1), (2, None)]


@pytest.mark.parametrize("loop,want", [((0, 0, 1), [(0, None), (1, None)]),
                                       ((0, 2, 1), [(0, 0), (1, None)]),
                                       ((1, 2, 3), [(0, None), (1, 0), (1, 1), (1, 2)]),
                                       ((0, 1, 2), [(0, 0), (0, 1), (1, None)])])
def test_layer_runs(loop, want):
    assert LusadraConfig.from_dict(R.make_config(layers=2, loop=loop)).layer_runs() == want


def test_config_reader_refuses_what_it_does_not_know():
    cfg = R.make_config()
    cfg["layers"][0]["type"] = "serial"
    with pytest.raises(ValueError):
        LusadraConfig.from_dict(cfg)
    cfg = R.make_config()
    cfg["layers"][1]["mlp"]["kind"] = "routed"
    with pytest.raises(ValueError):
        LusadraConfig.from_dict(cfg)
    cfg = R.make_config(loop=(1, 0, 1))
    with pytest.raises(ValueError):
        LusadraConfig.from_dict(cfg)


def test_registry():
    assert {"Lusadra", "LlamaDecodeStack"} <= set(registry.supported_architectures())
    model_cls, config_cls = registry.resolve("Lusadra")
    assert model_cls.__name__ == "LusadraForCausalLM" and config_cls is LusadraConfig
    with pytest.raises(ValueError):
        registry.resolve("NoSuchModel")
    assert registry.architecture_of({"architectures": ["X"]}) == "X"


def test_safetensors_reader_round_trip(tmp_path):
    cfg = R.make_config()
    W = R.make_weights(cfg, seed=3)
    W["table"] = torch.arange(12, dtype=torch.int32).reshape(3, 4)
    R.write_checkpoint(str(tmp_path), cfg, W)
    got = load_safetensors(str(tmp_path / "model.safetensors"))
    assert set(got) == set(W)
    for k in W:
        assert got[k].dtype == W[k].dtype and got[k].shape == W[k].shape and torch.equal(got[k], W[k]), k


def test_safetensors_reader_checks_offsets(tmp_path):
    import struct
    h = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 12]}}).encode()
    (tmp_path / "m.safetensors").write_bytes(struct.pack("<Q", len(h)) + h + b"\0" * 16)
    with pytest.raises(ValueError):
        load_safetensors(str(tmp_path / "m.safetensors"))


def test_cache_manager_reuses_blocks_and_slots():
    c = CacheManager(num_blocks=6, block_size=4, num_slots=2)
    s0 = c.admit("a")
    t = list(c.grow("a", 9))
    assert len(t) == 3 and c.free_blocks == 3
    assert c.grow("a", 12) == t and len(c.grow("a", 13)) == 4
    s1 = c.admit("b")
    assert s1 != s0 and not c.can_admit(1)          # no slot left
    with pytest.raises(RuntimeError):
        c.grow("b", 9)                               # 3 blocks needed, 2 free
    c.grow("b", 8)
    c.free("a")
    assert c.free_blocks == 4 and c.free_slots == 1
    assert c.admit("c") == s0                        # the slot that came back is used again
    again = c.grow("c", 16)
    assert set(again) == set(c.block_table("c")) and set(again) <= set(range(6))
    assert set(again) == set(range(6)) - set(c.block_table("b"))
    with pytest.raises(KeyError):
        c.admit("c")


def test_sequence_batch_build():
    b = SequenceBatch.build([3, 1], [5, 0], [[7, 2], [4]], [1, 0], 4, "cpu")
    assert b.positions.tolist() == [5, 6, 7, 0]
    assert b.slot_mapping.tolist() == [2 * 4 + 1, 2 * 4 + 2, 2 * 4 + 3, 4 * 4]
    assert b.token_seq.tolist() == [0, 0, 0, 1] and b.query_start_loc.tolist() == [0, 3, 4]
    assert b.block_tables.tolist() == [[7, 2], [4, 0]] and b.state_slots.tolist() == [1, 0]
    assert (b.max_query_len, b.max_seq_len) == (3, 8)
    with pytest.raises(AssertionError):
        SequenceBatch.build([6], [0], [[1]], [0], 4, "cpu")


def _seq(name, n, max_tokens=4):
    return Sequence(name, list(range(1, n + 1)), SamplingParams(max_tokens=max_tokens))


def _advance(step):
    for s, n in step:
        s.num_computed += n
        if s.num_computed == len(s):
            s.output_token_ids.append(0)


def test_scheduler_cuts_prompts_and_puts_decodes_first():
    cache = CacheManager(64, 4, 3)
    sch = Scheduler(cache, max_num_batched_tokens=10)
    a, b = _seq("a", 14), _seq("b", 3)
    sch.add(a)
    sch.add(b)
    s1 = sch.schedule()
    assert [(s.seq_id, n) for s, n in s1] == [("a", 10)]
    _advance(s1)
    s2 = sch.schedule()
    assert [(s.seq_id, n) for s, n in s2] == [("a", 4), ("b", 3)]
    _advance(s2)
    s3 = sch.schedule()
    assert [(s.seq_id, n) for s, n in s3] == [("a", 1), ("b", 1)]
    _advance(s3)
    sch.finish(a, "length")
    assert not cache.is_live("a") and cache.is_live("b")
    c = _seq("c", 30)
    sch.add(c)
    s4 = sch.schedule()
    assert [(s.seq_id, n) for s, n in s4] == [("b", 1), ("c", 9)]


def test_scheduler_preempts_the_newest_when_blocks_run_out():
    cache = CacheManager(num_blocks=4, block_size=4, num_slots=2)
    sch = Scheduler(cache, max_num_batched_tokens=64)
    a, b = _seq("a", 8, 8), _seq("b", 7, 8)
    sch.add(a)
    sch.add(b)
    _advance(sch.schedule())                      # a: 2 blocks, b: 2 blocks, pool empty
    step = sch.schedule()                         # a needs a third block: b gives way
    assert [(s.seq_id, n) for s, n in step] == [("a", 1)]
    assert sch.num_preemptions == 1 and b.num_computed == 0 and sch.waiting[0] is b
    assert not cache.is_live("b") and cache.free_slots == 1
    _advance(step)
    sch.finish(a, "stop")
    step = sch.schedule()                         # b starts over with its prompt and its one token
    assert [(s.seq_id, n) for s, n in step] == [("b", 8)]


def test_scheduler_refuses_what_can_never_fit():
    sch = Scheduler(CacheManager(2, 4, 1))
    with pytest.raises(ValueError):
        sch.add(_seq("a", 8, 4))


def test_sampler():
    logits = torch.tensor([[0.0, 3.0, 1.0, 2.9], [5.0, 0.0, 0.0, 0.0]])
    s = Sampler()
    assert s(logits, [SamplingParams(), SamplingParams()], [None, None]) == [1, 0]
    g = torch.Generator().manual_seed(0)
    p = SamplingParams(temperature=1.0, top_k=2)
    seen = {s(logits[:1], [p], [g])[0] for _ in range(60)}
    assert seen == {1, 3}
    p = SamplingParams(temperature=1.0, top_p=0.4)       # the most likely token alone passes 0.4
    assert {s(logits[:1], [p], [g])[0] for _ in range(20)} == {1}
    a = s(logits, [SamplingParams(temperature=2.0, seed=1)] * 2, [torch.Generator().manual_seed(1)] * 2)
    b = s(logits, [SamplingParams(temperature=2.0, seed=1)] * 2, [torch.Generator().manual_seed(1)] * 2)
    assert a == b
    with pytest.raises(ValueError):
        SamplingParams(top_p=0.0)


def test_oracle_mechanisms_agree_with_their_closed_forms():
    """The reference itself: a window of one attends to itself only; with no decay change
    (ln a = 0) the linear attention is a running sum; PolyNorm of a constant row."""
    torch.manual_seed(0)
    n, H, D = 5, 2, 4
    q, k = torch.randn(n, H * D, dtype=R.F), torch.randn(n, D, dtype=R.F)
    out = R.windowed_key_attention(q, k, torch.arange(n), H, 1, D, 1, 0.3, 0.2, 2, R.head_slopes(H))
    assert torch.allclose(out.view(n, H, D), k[:, None, :].expand(n, H, D))
    qq, kk, vv = torch.randn(n, D, dtype=R.F), torch.randn(n, D, dtype=R.F), torch.randn(n, 3, dtype=R.F)
    o, S = R.gated_linear_attention(qq, kk, vv, torch.zeros(n, D, dtype=R.F), 1, D, 3)
    want = torch.stack([sum((qq[t] @ kk[s]) * vv[s] for s in range(t + 1)) for t in range(n)])
    assert torch.allclose(o[:, 0], want) and torch.allclose(S[0], kk.T @ vv)
    z = torch.full((1, 8), 2.0, dtype=R.F)
    assert torch.allclose(R.poly_norm(z, [1.0, 1.0, 1.0, 0.5], 0.0), torch.full((1, 8), 3.5, dtype=R.F))


def test_scheduler_unblocks_prompts_that_starve_each_other():
    cache = CacheManager(num_blocks=4, block_size=4, num_slots=2)
    sch = Scheduler(cache, max_num_batched_tokens=6)
    a, b = _seq("a", 11, 2), _seq("b", 11, 2)
    sch.add(a)
    sch.add(b)
    _advance(sch.schedule())          # a: 6 tokens, 2 blocks
    _advance(sch.schedule())          # a: 5 more (3 blocks), b: 1 token (1 block) -> pool empty
    for _ in range(12):
        step = sch.schedule()
        assert step, "the scheduler stalled with work left"
        _advance(step)
        for s, _n in step:
            if len(s.output_token_ids) >= 2 and not s.finished:
                sch.finish(s, "length")
        if not sch.has_unfinished():
            break
    assert a.finished and b.finished and cache.free_blocks == 4
