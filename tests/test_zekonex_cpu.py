"""Zekonex without a GPU: configuration, the model as data (tensor names, running order, cache
needs), and the plain model against itself (a sequence fed whole and in portions)."""

import numpy as np
import pytest
import torch

import plain_zekonex as pz
import tiny_zekonex as tz
from mini_infer_amd.exceptions import ConfigError
from mini_infer_amd.models import architecture_for


def model_of(cfg, dtype=torch.bfloat16):
    arch = architecture_for(cfg)
    return arch.make_model(arch.parse_config(cfg), dtype, "cpu")


@pytest.mark.parametrize("name", sorted(tz.CONFIGS))
def test_the_model_asks_for_exactly_the_checkpoints_tensors(name):
    cfg, _ = tz.CONFIGS[name]
    specs = model_of(cfg).param_specs()
    assert {k: tuple(v.shape) for k, v in specs.items()} == tz.tensor_shapes(cfg)
    # what enters a recurrence or a norm stays 32-bit whatever the engine's dtype
    for leaf in ("mix.A_log", "mix.dt_bias", "mix.norm", "mix.q.conv", "mix.dkv.norm", "mlp.up.b"):
        assert all(v.dtype == "float32" for k, v in specs.items() if k.endswith(leaf))


def test_the_running_order_repeats_the_looped_stretch_and_marks_each_pass():
    cfg, _ = tz.CONFIGS["A"]  # layers 0..1 three times, then 2, 3
    order = model_of(cfg).spec.order
    assert [c.layer for c in order] == [0, 1, 0, 1, 0, 1, 2, 3]
    assert [c.stream_add for c in order] == [("loop.step", 0), None, ("loop.step", 1), None, ("loop.step", 2), None, None, None]
    assert [run for run in pz.layer_runs(cfg)] == [(0, 0), (1, None), (0, 1), (1, None), (0, 2), (1, None), (2, None), (3, None)]
    cfg_b, _ = tz.CONFIGS["B"]
    assert [c.layer for c in model_of(cfg_b).spec.order] == [0, 1, 2, 2, 3, 4]
    no_loop, _ = tz.CONFIGS["C"]
    assert all(c.stream_add is None for c in model_of(no_loop).spec.order) and "loop.step" not in model_of(no_loop).param_specs()


def test_every_pass_of_a_loop_has_caches_and_state_of_its_own():
    cfg, block = tz.CONFIGS["A"]
    needs = model_of(cfg).cache_needs(block)
    assert len(needs) == 8 and all(need is not None for need in needs)
    first = needs[0].state
    assert first["recurrent"].shape == (4, 20, 64) and first["recurrent"].dtype == torch.float32
    assert first["tail"].shape == (2, 2 * 4 * 12 + 4 * 20) and first["tail"].dtype == torch.bfloat16
    assert needs[2].state == first and needs[4].state == first
    pages = needs[1].pages  # attention: keys of 16, values of 24
    assert (pages.num_kv_heads, pages.head_dim, pages.value_dim, pages.window) == (2, 16, 24, None)
    latent = needs[6].pages  # one row [latent | rotated part] per token, no value pages
    assert (latent.num_kv_heads, latent.head_dim, latent.value_dim) == (1, 22 + 6, 0)
    one_tap = model_of(tz.CONFIGS["B"][0]).cache_needs(8)[1].state
    assert set(one_tap) == {"recurrent"}  # a convolution of one tap has nothing to carry
    assert all(need.pages is None for need in model_of(tz.CONFIGS["D"][0]).cache_needs(4))


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=4), "rot_dim"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "mlp"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["loop"].update(times=0), "loop.times"),
    (lambda c: c.pop("residual_mult"), "residual_mult"),
    (lambda c: c["norm"].update(eps=0), "eps"),
])
def test_configurations_the_design_does_not_have_are_refused(change, message):
    import copy

    cfg = copy.deepcopy(tz.CONFIGS["A"][0])
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        architecture_for(cfg).parse_config(cfg)


@pytest.mark.parametrize("name", sorted(tz.CONFIGS))
def test_the_plain_model_gives_the_same_logits_whole_and_in_portions(name):
    cfg, _ = tz.CONFIGS[name]
    weights = {k: v.astype(np.float64) for k, v in tz.make_weights(cfg, seed=3).items()}
    tokens = tz.random_tokens(cfg, 23, seed=4)
    model = pz.PlainZekonex(cfg, weights)
    whole = model.forward(tokens)
    memory: dict = {}
    parts = [model.forward(tokens[a:b], memory) for a, b in ((0, 1), (1, 3), (3, 4), (4, 15), (15, 23))]
    np.testing.assert_allclose(np.concatenate(parts), whole, rtol=0, atol=1e-10)
    assert np.abs(whole).max() > 0.5  # (not a model whose logits say nothing)
