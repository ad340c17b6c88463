"""Gilidra's configuration on the CPU: reading, the layers as data, the run order, the declared tensors."""
import copy
import json

import pytest

import gilidra_helpers as G
import vipera_rs_amd  # noqa: F401
from vipera_rs_amd.config import GilidraConfig, config_from_dict, load_config
from vipera_rs_amd.errors import InvalidArgumentError, UnsupportedError
from vipera_rs_amd.models import declare_cache_needs, declare_model


def test_the_architecture_is_found_by_its_name_and_layers_become_parts():
    cfg = config_from_dict(G.written_config(G.G1))
    assert isinstance(cfg, GilidraConfig) and cfg.vocab_size == 211 and cfg.hidden_size == 96
    specs = cfg.layer_specs()
    assert [s.mixer.kind for s in specs] == ["latent_attention", "wkv", "gated_delta", "latent_attention", "gated_delta"]
    assert [s.ffn.kind for s in specs] == ["moe", "moe", "none", "moe", "moe"]
    assert all(s.block == "parallel" and s.mixer_norm.kind == "dyt" for s in specs)
    assert [s.position.kind for s in specs] == ["rotary_neox", "none", "none", "rotary_neox", "none"]
    assert [(e.layer, e.cache_of) for e in cfg.schedule()] == [(0, None), (1, None), (2, None), (3, 0), (4, None)]
    assert cfg.head_spec().params["scale"] == 0.5 and cfg.embedding_spec().params["norm"].kind == "dyt"
    assert GilidraConfig.from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_a_shared_cache_keeps_the_widest_window_of_its_readers():
    cfg = config_from_dict(G.written_config(G.G1))
    first, second = cfg.layer_specs()[0].mixer.params, cfg.layer_specs()[3].mixer.params
    assert (first["window"], second["window"]) == (13, 29) and first["retain"] == second["retain"] == 29
    assert second["shares_cache"] and not first["shares_cache"]
    needs = declare_cache_needs(cfg)
    assert needs[3].owner == 0 and needs[0].kv == needs[3].kv and needs[0].kv.window == 29 and needs[0].kv.head_dim == 64
    assert needs[1].kv is None and needs[1].state.shape == (3 * 256 + 96,)     # a head's 16 x 16 matrix, then the last h
    # heads of 16 x 24 padded to two value tiles of 16, then three rows of the convolution's inputs
    assert needs[2].state.shape == (4 * 2 * 256 + 3 * (2 * 2 * 16 + 4 * 24),)
    # one reader without a window: everything is kept
    other = config_from_dict(G.written_config(G.G2))
    assert [s.mixer.params.get("retain") for s in other.layer_specs() if s.mixer.kind == "latent_attention"] == [0, 0]
    assert other.layer_specs()[3].mixer.params["window"] == 7 and other.head_spec().params["scale"] == 1.0


def test_declared_tensors_are_the_folders(tmp_path):
    folder = G.make_folder(tmp_path / "m", G.G1, 3)
    cfg = load_config(folder)
    declared = {s.name: s.shape for s in declare_model(cfg)}
    made = G.make_weights(G.G1, 3)
    assert set(declared) == set(made)
    for name, shape in declared.items():
        assert all(w == -1 or w == f for w, f in zip(shape, made[name].shape)) and len(shape) == made[name].dim(), name
    assert declared["l1.mix.w1"] == (-1, 96)           # the decay's rank is whatever the folder stores
    assert "l3.mix.dkv" not in declared and "l2.mlp.router" not in declared


@pytest.mark.parametrize("change, error", [
    (lambda c: c["layers"][3]["mixer"].update(kv_from=2), InvalidArgumentError),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), InvalidArgumentError),
    (lambda c: c["layers"][3]["mixer"].update(kv_rank=48), InvalidArgumentError),
    (lambda c: c["layers"][0].update(type="conv"), UnsupportedError),
    (lambda c: c["layers"][2]["mixer"].update(kv_heads=3), InvalidArgumentError),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), InvalidArgumentError),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=5), InvalidArgumentError),
    (lambda c: c.pop("norm"), InvalidArgumentError),
    (lambda c: c.pop("vocab"), InvalidArgumentError),
])
def test_a_bad_configuration_is_refused_with_its_key(change, error):
    data = copy.deepcopy(G.written_config(G.G1))
    change(data)
    with pytest.raises(error):
        config_from_dict(data)


def test_the_command_line_reads_the_model(tmp_path, capsys):
    from vipera_rs_amd.cli import main

    folder = G.make_folder(tmp_path / "m", G.G2, 5)
    assert main(["model-info", folder]) == 0
    shown = capsys.readouterr().out
    assert "Gilidra" in shown
