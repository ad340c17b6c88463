"""Zulesun's configuration on the CPU: reading, the layers as data, the declared tensors, what a request keeps; and
the plain implementation's mechanisms against closed forms of their own."""
import copy

import numpy as np
import pytest

import vipera_rs_amd  # noqa: F401
import zulesun_helpers as Z
from plain import zulesun_plain as P
from vipera_rs_amd.config import ZulesunConfig, config_from_dict, load_config
from vipera_rs_amd.errors import InvalidArgumentError, UnsupportedError
from vipera_rs_amd.models import declare_cache_needs, declare_model


def test_the_architecture_is_found_by_its_name_and_layers_become_parts():
    cfg = config_from_dict(Z.Z1)
    assert isinstance(cfg, ZulesunConfig) and cfg.vocab_size == 131 and cfg.hidden_size == 48
    specs = cfg.layer_specs()
    assert [s.mixer.kind for s in specs] == ["mixer_pair", "decay_attention", "mixer_pair", "decay_attention"]
    assert [s.ffn.kind for s in specs] == ["moe", "mlp", "none", "moe"]
    assert all(s.block == "sandwich_norm" and s.mixer_norm.params["one_plus"] for s in specs)
    assert all(s.extras["after"].kind == "token_side" and s.extras["after"].params["index"] == i for i, s in enumerate(specs))
    assert [s.position.kind for s in specs] == ["rotary_neox", "none", "rotary_neox", "none"]
    first = specs[0].mixer.params
    assert (first["left_scale"], first["right_scale"]) == (0.7, 1.3)
    attention = first["left"].params
    assert (attention["chunk"], attention["softcap"], attention["value_dim"], attention["head_dim"]) == (13, 5.0, 24, 16)
    assert specs[0].position.params["scaling_factor"] == 4.0 and specs[2].position.params["scaling_factor"] == 1.0
    assert specs[2].mixer.params["left"].params["softcap"] == 0.0
    router = specs[0].ffn.params
    assert (router["groups"], router["keep"], router["scores"], router["limit"], router["alpha"]) == (3, 2, "all", None, 1.0)
    assert specs[3].ffn.params["groups"] == 1
    assert cfg.embedding_spec().params["side"] == {"tensor": "side.embed", "width": 24}
    assert ZulesunConfig.from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    other = config_from_dict(Z.Z2)
    assert "after" not in other.layer_specs()[0].extras and "side" not in other.embedding_spec().params
    assert other.layer_specs()[1].position.kind == "none" and other.layer_specs()[1].mixer.params["left"].params["chunk"] == 0


def test_what_a_request_keeps():
    needs = declare_cache_needs(config_from_dict(Z.Z1))
    assert needs[1].kv is None and needs[3].kv is None
    # keys of 16 beside values of 24 share pages of the wider width, rounded up to a multiple of 16; blocks of
    # positions keep everything
    assert (needs[0].kv.kv_heads, needs[0].kv.head_dim, needs[0].kv.window) == (2, 32, 0)
    assert (needs[2].kv.kv_heads, needs[2].kv.head_dim, needs[2].kv.window) == (1, 32, 0)
    # 40 channels of 12 numbers (padded to 16), then two rows of the convolution's inputs
    assert needs[0].state.shape == (40 * 16 + 2 * 40,)
    # three heads: 8 value channels of 24 key channels, padded to 32
    assert needs[1].state.shape == (3 * 8 * 32,)
    assert needs[3].state.shape == (20 * 64,)


def test_declared_tensors_are_the_folders(tmp_path):
    for made_from in (Z.Z1, Z.Z2):
        folder = Z.make_folder(tmp_path / f"m{made_from['vocab']}", made_from, 3)
        declared = {s.name: tuple(s.shape) for s in declare_model(load_config(folder)) if not s.optional}
        made = {name: tuple(t.shape) for name, t in Z.make_weights(made_from, 3).items()}
        assert declared == made
    optional = {s.name for s in declare_model(config_from_dict(Z.Z1)) if s.optional}
    assert optional == {"l2.norm2", "l2.norm2b"}      # a layer without a feed-forward does not need the norms around it


@pytest.mark.parametrize("change, error", [
    (lambda c: c["layers"][0].update(type="conv"), UnsupportedError),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5]), InvalidArgumentError),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), InvalidArgumentError),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=5), InvalidArgumentError),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=32), InvalidArgumentError),
    (lambda c: c["layers"][0]["mixer"]["right"].pop("state"), InvalidArgumentError),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), InvalidArgumentError),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), InvalidArgumentError),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=1, count=6), InvalidArgumentError),
    (lambda c: c["layers"][1]["mlp"].update(kind="gated"), UnsupportedError),
    (lambda c: c.pop("norm"), InvalidArgumentError),
    (lambda c: c.pop("vocab"), InvalidArgumentError),
])
def test_a_bad_configuration_is_refused_with_its_key(change, error):
    data = copy.deepcopy(Z.Z1)
    change(data)
    with pytest.raises(error):
        config_from_dict(data)


def test_the_command_line_reads_the_model(tmp_path, capsys):
    from vipera_rs_amd.cli import main

    folder = Z.make_folder(tmp_path / "m", Z.Z2, 5)
    assert main(["model-info", folder]) == 0
    assert "Zulesun" in capsys.readouterr().out


# --- the plain implementation against closed forms ------------------------------------------------------------------
def test_plain_linear_attention_is_its_unrolled_sum():
    rng = np.random.default_rng(0)
    p = {"heads": 2, "dim": 5, "vdim": 3, "decay": [0.8, 0.95]}
    w = {"q": rng.standard_normal((10, 7)), "k": rng.standard_normal((10, 7)), "v": rng.standard_normal((6, 7)),
         "g": rng.standard_normal((6, 7)), "o": np.eye(6), "norm": np.ones(6)}
    h = rng.standard_normal((9, 7))
    got = P.lightning(h, w, p, 1e-5)
    q, k, v = (P.silu(h @ w[n].T) for n in "qkv")
    o = np.zeros((9, 6))
    for head, decay in enumerate(p["decay"]):
        qs, ks, vs = q[:, 5 * head:5 * head + 5], k[:, 5 * head:5 * head + 5], v[:, 3 * head:3 * head + 3]
        for t in range(9):
            for s in range(t + 1):
                o[t, 3 * head:3 * head + 3] += decay ** (t - s) * (qs[t] @ ks[s]) * vs[s]
    want = P.norm_plain(o, w["norm"], 1e-5) * P.sigmoid(h @ w["g"].T)
    assert np.allclose(got, want, rtol=1e-10, atol=1e-12)


def test_plain_attention_blocks_and_rotation():
    rng = np.random.default_rng(1)
    base = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 3, "scale": 0.5, "rot": {"base": 100.0, "dims": 4}}
    w = {"q": rng.standard_normal((8, 6)), "k": rng.standard_normal((4, 6)), "v": rng.standard_normal((3, 6)),
         "g": rng.standard_normal((6, 6)), "o": np.eye(6), "q.norm": np.ones(8), "k.norm": np.ones(4)}
    h = rng.standard_normal((10, 6))
    whole = P.chunked_attention(h, w, base, 1e-5)
    blocks = P.chunked_attention(h, w, dict(base, mask={"size": 4}), 1e-5)
    # a token at the start of a block sees itself only: its output is its own value, gated
    v = h @ w["v"].T
    gate = P.sigmoid(h @ w["g"].T)
    for t in (0, 4, 8):
        assert np.allclose(blocks[t], np.tile(v[t], 2) * gate[t])
    assert np.allclose(blocks[:4], whole[:4]) and not np.allclose(blocks[5], whole[5])
    # the rotation depends on the distance only: the same tokens four positions later, inside one block of eight
    eight = P.chunked_attention(h[:4], w, dict(base, mask={"size": 8}), 1e-5, first_position=4)
    assert np.allclose(eight, whole[:4])
    # scaled frequencies: a factor of two is half the position
    scaled = dict(base, rot={"base": 100.0, "dims": 4, "scaling": {"factor": 2.0}})
    x = rng.standard_normal((3, 1, 4))
    assert np.allclose(P.rotate_half(x, np.array([2.0, 4.0, 6.0]), 4, 100.0, 2.0), P.rotate_half(x, np.array([1.0, 2.0, 3.0]), 4, 100.0, 1.0))
    assert scaled["rot"]["scaling"]["factor"] == 2.0
    # a cap bounds the scores
    capped = P.chunked_attention(h, w, dict(base, scale=50.0, softcap=1.0), 1e-5)
    assert np.isfinite(capped).all() and not np.allclose(capped, P.chunked_attention(h, w, dict(base, scale=50.0), 1e-5))


def test_plain_routing_keeps_the_best_groups():
    scores = np.array([0.05, 0.30, 0.02, 0.03, 0.25, 0.24, 0.06, 0.05])
    assert P.route(scores, 2, 1, 1) == [1, 4]
    assert P.route(scores, 2, 4, 1) == [1, 0]            # the best group is (0, 1)
    assert P.route(scores, 3, 4, 2) == [1, 4, 5]         # groups (0, 1) and (4, 5)
    assert P.route(scores, 2, 2, 1) == [1, 0]            # halves: the first holds the largest score
    tie = np.array([0.25, 0.25, 0.25, 0.25])
    assert P.route(tie, 2, 2, 1) == [0, 1]


def test_plain_selective_scan_with_one_tap_and_no_decay_is_a_running_sum():
    rng = np.random.default_rng(2)
    p = {"inner": 3, "state": 2, "dt_rank": 2, "conv": 1}
    w = {"in": rng.standard_normal((6, 4)), "conv": np.ones((3, 1)), "conv.b": np.zeros(3), "x": rng.standard_normal((6, 3)),
         "dt": rng.standard_normal((3, 2)), "dt.b": np.zeros(3), "A_log": np.full((3, 2), -40.0), "D": np.zeros(3),
         "o": np.eye(3)}
    h = rng.standard_normal((6, 4))
    got = P.selective_scan(h, w, p)
    xz = h @ w["in"].T
    x, z = P.silu(xz[:, :3]), xz[:, 3:]
    low = x @ w["x"].T
    dt = P.softplus(low[:, :2] @ w["dt"].T)
    state = np.cumsum((dt * x)[:, :, None] * low[:, None, 2:4], axis=0)
    want = np.einsum("tcn,tn->tc", state, low[:, 4:6]) * P.silu(z)
    assert np.allclose(got, want, rtol=1e-9, atol=1e-12)
