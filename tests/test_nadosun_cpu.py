"""Nadosun without a GPU: configuration, the model as data, tensor names, and the plain model's own
consistency (portions against whole prompts, what a window hides, what the state carries)."""

import copy

import numpy as np
import pytest
import torch

import plain_nadosun as pn
import tiny_nadosun as tn


def _model(cfg, dtype=torch.bfloat16):
    from mini_infer_amd.models import architecture_for

    arch = architecture_for(cfg)
    return arch, arch.make_model(arch.parse_config(cfg), dtype, "cpu")


@pytest.mark.parametrize("name", sorted(tn.CONFIGS))
def test_the_model_asks_for_exactly_the_tensors_of_a_checkpoint(name):
    cfg, _ = tn.CONFIGS[name]
    _, model = _model(cfg)
    specs = model.param_specs()
    shapes = tn.tensor_shapes(cfg)
    assert set(specs) == set(shapes)
    assert all(tuple(specs[k].shape) == tuple(shapes[k]) for k in shapes)
    # gains, scales, biases, norm weights and activation coefficients stay 32-bit in both engines
    narrow = {k for k, s in specs.items() if s.dtype == "compute"}
    assert all(k.endswith((".q", ".k", ".o", ".z", ".x", ".g", ".up", ".down", ".gate", ".proj", "embed", "head"))
               or k.endswith("side.norm") for k in narrow)
    assert specs["l0.norm1"].dtype == "float32" and specs["l0.ls1"].dtype == "float32"


def test_the_architecture_is_chosen_by_either_key_of_the_configuration():
    from mini_infer_amd.models import architecture_for

    cfg = copy.deepcopy(tn.TINY_S)
    assert architecture_for(cfg).name == "Nadosun"
    del cfg["architecture"]
    cfg["architectures"] = ["Nadosun"]
    assert architecture_for(cfg).name == "Nadosun"
    with pytest.raises(ValueError):
        architecture_for({"architecture": "NoSuchModel"})


def test_cache_needs_follow_the_layers():
    from mini_infer_amd.cache.manager import CacheManager

    cfg, block = tn.CONFIGS["P"]
    _, model = _model(cfg)
    needs = model.cache_needs(block)
    assert [n.pages is not None for n in needs] == [True, False, False, True]
    assert needs[1].state.shape == (80,) and needs[2].state.shape == (48,) and needs[1].state.dtype == torch.float32
    assert needs[0].pages.window == 24 and needs[3].pages.window == 7 and needs[3].pages.num_kv_heads == 1
    manager = CacheManager(needs, page_size=block, num_pages=8, max_requests=2, allocate_storage=False)
    assert len(manager.groups) == 2  # two attention layers of different shape: a page group each
    _, no_pages = _model(tn.TINY_S)
    assert not CacheManager(no_pages.cache_needs(4), page_size=4, num_pages=1, max_requests=2, allocate_storage=False).has_pages


@pytest.mark.parametrize(
    "change, message",
    [
        (lambda c: c["layers"][0].update(type="conv"), "type"),
        (lambda c: c["layers"][0]["mixer"].update(vdim=12), "vdim"),
        (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
        (lambda c: c["layers"][0]["mixer"].pop("mask"), "mask"),
        (lambda c: c["layers"][1]["mixer"].update(width=0), "width"),
        (lambda c: c["layers"][0].update(mlp={"kind": "routed", "ff": 8}), "mlp"),
        (lambda c: c.pop("token_side"), "token_side"),
        (lambda c: c["norm"].update(eps=0.0), "eps"),
        (lambda c: c.update(layers=[]), "layers"),
        (lambda c: c["embedding"].update(scale="big"), "scale"),
    ],
)
def test_a_configuration_that_the_design_does_not_have_is_refused(change, message):
    from mini_infer_amd.exceptions import ConfigError
    from mini_infer_amd.models.nadosun import NadosunConfig

    cfg = copy.deepcopy(tn.TINY_P)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        NadosunConfig.from_dict(cfg)


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    from mini_infer_amd.weights import CheckpointReader, write_random_model
    from mini_infer_amd.weights.loader import check_names_and_shapes

    folder = write_random_model(tn.TINY_Q, 3, tmp_path / "m")
    reader = CheckpointReader(folder)
    _, model = _model(tn.TINY_Q)
    check_names_and_shapes(model.param_specs(), model.optional_names(), reader.shapes)
    assert reader.shapes["final.norm"] == () and reader.shapes["l1.mlp.act"] == (4,)


# -- the plain model against itself ------------------------------------------------------------


@pytest.mark.parametrize("name", ["P", "Q", "S"])
def test_plain_model_portions_give_what_the_whole_prompt_gives(name):
    cfg, _ = tn.CONFIGS[name]
    weights = tn.make_weights(cfg, 5)
    tokens = tn.random_tokens(cfg, 37, seed=1)
    whole = pn.logits(cfg, weights, tokens)
    for cuts in ([1] * 37, [2, 7, 2, 13, 3, 2, 8], [30, 7], [36, 1]):
        np.testing.assert_allclose(pn.logits(cfg, weights, tokens, cuts=cuts), whole, rtol=0, atol=1e-9)


def test_plain_window_hides_exactly_the_keys_beyond_it():
    """Changing a token changes the attention output of the positions whose window holds it and of no other
    (one attention layer alone: no recurrence carries the change further)."""
    cfg = tn.config(50, 32, [tn.attention(2, 1, 8, 6, 0.8)], scale=1.0, eps=1e-6, side=4)
    weights = tn.make_weights(cfg, 11)
    rng = np.random.default_rng(0)
    h = rng.standard_normal((20, 32))
    base, _, _ = pn.windowed_attention(h, weights, "l0.mix.", cfg["layers"][0]["mixer"], 1e-6)
    h2 = h.copy()
    h2[4] += 1.0
    moved, _, _ = pn.windowed_attention(h2, weights, "l0.mix.", cfg["layers"][0]["mixer"], 1e-6)
    changed = np.abs(moved - base).max(axis=1) > 1e-12
    assert changed.tolist() == [4 <= i < 4 + 6 for i in range(20)]


def test_plain_recurrence_carries_its_state_and_starts_from_zero():
    cfg = tn.TINY_S
    weights = tn.make_weights(cfg, 2)
    h = np.random.default_rng(3).standard_normal((9, cfg["width"]))
    whole, last = pn.min_gru(h, weights, "l0.mix.")
    first, carried = pn.min_gru(h[:4], weights, "l0.mix.")
    second, end = pn.min_gru(h[4:], weights, "l0.mix.", carried)
    np.testing.assert_allclose(np.concatenate([first, second]), whole, atol=1e-12)
    np.testing.assert_allclose(end, last, atol=1e-12)
    lost, _ = pn.min_gru(h[4:], weights, "l0.mix.")  # a lost state shows
    assert np.abs(lost - whole[4:]).max() > 1e-3
    # the candidate's two branches meet at zero with equal value and slope
    u = np.array([-1e-9, 0.0, 1e-9])
    np.testing.assert_allclose(np.where(u >= 0, u + 0.5, pn.sigmoid(u)), 0.5, atol=1e-9)


def test_plain_sinusoid_interleaves_sine_and_cosine_also_at_an_odd_width():
    wave = pn.sinusoid(np.array([0, 3]), 7)
    assert wave.shape == (2, 7)
    np.testing.assert_allclose(wave[0], [0, 1, 0, 1, 0, 1, 0], atol=1e-15)
    f = 10000.0 ** (-2.0 * 2 / 7)
    np.testing.assert_allclose(wave[1, 4:6], [np.sin(3 * f), np.cos(3 * f)], atol=1e-15)
    np.testing.assert_allclose(wave[1, 6], np.sin(3 * 10000.0 ** (-2.0 * 3 / 7)), atol=1e-15)


def test_plain_poly_norm_is_its_three_normed_powers():
    z = np.random.default_rng(1).standard_normal((3, 11))
    got = pn.poly_norm(z, np.array([2.0, -1.0, 0.5, 0.25]), 1e-6)
    want = 2.0 * z / np.sqrt((z**2).mean(1, keepdims=True) + 1e-6) - z**2 / np.sqrt((z**4).mean(1, keepdims=True) + 1e-6) \
        + 0.5 * z**3 / np.sqrt((z**6).mean(1, keepdims=True) + 1e-6) + 0.25
    np.testing.assert_allclose(got, want, atol=1e-12)
