"""Dopipel's configuration reader, layer runs, checkpoint names and cache shapes (no GPU), and the
float64 reference against itself: a prompt's logits do not depend on what follows a position."""
import torch

from tests import dopipel_oracle as R
from vllm_legacy_amd.model.dopipel import DopipelConfig, DopipelForCausalLM
from vllm_legacy_amd.model.registry import resolve, supported_architectures


def small():
    return R.make_config([R.mingru_layer(24, R.dense_mlp(40)), R.attention_layer(4, 2, 8, vdim=12, rot_dims=4, mlp=R.moe_mlp(3, 1, 2, 10, 6)),
                          R.attention_layer(2, 2, 8, mlp=None)], vocab=50, width=32, taps=3, loop=(1, 3, 2))


def test_registry_and_config():
    assert "Dopipel" in supported_architectures()
    model_cls, config_cls = resolve("Dopipel")
    assert model_cls is DopipelForCausalLM and config_cls is DopipelConfig
    cfg = DopipelConfig.from_dict(small())
    assert cfg.layer_runs() == [(0, None), (1, 0), (2, None), (1, 1), (2, None)]
    a = cfg.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims, a.interleaved) == (4, 2, 8, 12, 4, True)
    m = cfg.layers[1].mlp
    assert (m.kind, m.experts, m.identity, m.top, m.ff, m.shared_ff) == ("moe", 3, 1, 2, 10, 6)
    assert cfg.layers[2].mlp is None and cfg.taps == 3


def test_checkpoint_names_and_cache_shapes():
    raw = small()
    cfg = DopipelConfig.from_dict(raw)
    model = DopipelForCausalLM(cfg, torch.float32, "cpu")
    W = R.make_weights(raw)
    assert {k: tuple(v.shape) for k, v in W.items()} == model.tensor_shapes()
    assert model.load_weights(W) == len(W)
    caches = model.allocate_caches(5, 4, 2)
    assert len(caches) == 5
    assert caches[0]["state"].shape == (2, 24) and caches[0]["conv"].shape == (2, 2, 32)
    assert caches[1]["keys"].shape == (5, 4, 2, 8) and caches[1]["values"].shape == (5, 4, 2, 12)
    assert caches[1]["keys"].data_ptr() != caches[3]["keys"].data_ptr()      # a pass has its own


def test_bad_configs_are_refused():
    import pytest
    raw = small()
    raw["layers"][0]["type"] = "lstm"
    with pytest.raises(ValueError):
        DopipelConfig.from_dict(raw)
    raw = small()
    raw["layers"][1]["mlp"]["router"]["top"] = 9
    with pytest.raises(ValueError):
        DopipelConfig.from_dict(raw)
    raw = small()
    raw["loop"]["stop"] = 7
    with pytest.raises(ValueError):
        DopipelConfig.from_dict(raw)


def test_reference_is_causal():
    raw = small()
    W = R.make_weights(raw, seed=1)
    toks = torch.randint(0, 50, (12, ), generator=torch.Generator().manual_seed(0)).tolist()
    full = R.forward(toks, raw, W)
    assert float((R.forward(toks[:7], raw, W) - full[:7]).abs().max()) < 1e-9
