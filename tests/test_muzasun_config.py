"""Muzasun's configuration on the CPU: reading, the layers as data, the declared tensors, what a request keeps; and
the plain implementation's mechanisms against closed forms of their own."""
import copy
import math

import numpy as np
import pytest

import muzasun_helpers as M
import vipera_rs_amd  # noqa: F401
from plain import muzasun_plain as P
from vipera_rs_amd.config import MuzasunConfig, config_from_dict, load_config
from vipera_rs_amd.errors import InvalidArgumentError, UnsupportedError
from vipera_rs_amd.models import declare_cache_needs, declare_model


def test_the_architecture_is_found_by_its_name_and_layers_become_parts():
    cfg = config_from_dict(M.stored(M.M1))
    assert isinstance(cfg, MuzasunConfig) and cfg.vocab_size == 131 and cfg.hidden_size == 48
    specs = cfg.layer_specs()
    assert [s.mixer.kind for s in specs] == ["matrix_memory", "attention", "gated_delta", "attention", "attention"]
    assert [s.ffn.kind for s in specs] == ["moe", "gated_mlp", "none", "moe", "gated_mlp"]
    assert all(s.block == "parallel" and s.params == {"residual_mult": 0.7} for s in specs)
    assert all(s.mixer_norm.kind == "dyt" and s.mixer_norm.params["name"] == "norm1" and s.ffn_norm.params["name"] == "norm2"
               for s in specs)
    assert [s.position.kind for s in specs] == ["none", "rotary_neox", "none", "none", "rotary_neox"]
    assert specs[1].position.params == {"head_dim": 16, "rotary_dim": 8, "base": 1000.0}
    # the first layer that says so keeps its values, the next blends with them, a layer that does not say so does neither
    assert [s.mixer.params.get("value_mix") for s in specs] == [None, "source", None, "blend", None]
    first = specs[1].mixer.params
    assert (first["head_dim"], first["value_dim"], first["scale"], first["qk_norm"], first["qkv_bias"], first["out_bias"]) == \
        (16, 24, 0.3, "head", True, True)
    assert specs[0].mixer.params["gate_cap"] == 8.0
    delta = specs[2].mixer.params
    assert (delta["decay"], delta["gate"], delta["decay_rank"], delta["gate_rank"], delta["conv"]) == ("channel", "sigmoid", -1, -1, 3)
    router = specs[0].ffn.params
    assert (router["scores"], router["weigh"], router["shared"], router["limit"], router["alpha"], router["top"]) == \
        ("sigmoid", "input", 16, None, 1.0, 2)
    assert specs[3].ffn.params["shared"] is None
    assert cfg.head_spec().params["scale"] == 2.0 and cfg.final_norm_spec().params["name"] == "final.norm"
    assert MuzasunConfig.from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_what_a_request_keeps():
    needs = declare_cache_needs(config_from_dict(M.stored(M.M1)))
    assert [n.kv is None for n in needs] == [True, False, True, False, False]
    # keys of 16 beside values of 24 share pages of the wider width, rounded up to a multiple of 16
    assert (needs[1].kv.kv_heads, needs[1].kv.head_dim, needs[1].kv.window) == (2, 32, 0)
    assert (needs[3].kv.kv_heads, needs[3].kv.head_dim) == (2, 32) and (needs[4].kv.kv_heads, needs[4].kv.head_dim) == (1, 16)
    # three heads: 16 value channels (8 padded) of 32 key channels (24 padded), and the normalizer and the running
    # maximum once per tile of eight value channels
    assert needs[0].state.shape == (3 * (16 * 32 + 2 * 32 + 2),)
    # four heads of 16 value channels x 16 key channels, then two rows of the convolution's 96 inputs
    assert needs[2].state.shape == (4 * 16 * 16 + 2 * 96,)


def test_declared_tensors_are_the_folders(tmp_path):
    for made_from in (M.M1, M.M2):
        folder = M.make_folder(tmp_path / f"m{made_from['vocab']}", made_from, 3)
        ranks = M.ranks_of(made_from)
        declared = {s.name: tuple(s.shape) for s in declare_model(load_config(folder)) if not s.optional}
        made = {name: tuple(t.shape) for name, t in M.make_weights(made_from, 3).items()}
        # a layer without a feed-forward need not hold the norm in front of it, and a layer that blends no values not
        # the number for it; the folders of the tests hold the first and not the second
        optional = {s.name for s in declare_model(load_config(folder)) if s.optional}
        assert set(made) - set(declared) <= optional
        for name, shape in declared.items():
            # the two-step projections' inner size is the folder's: no key of the configuration gives it
            want = tuple(made[name][k] if d == -1 else d for k, d in enumerate(shape))
            assert made[name] == want, name
            if -1 in shape:
                layer = int(name.split(".")[0][1:])
                assert made[name][shape.index(-1)] in ranks[layer]
    optional = {s.name for s in declare_model(config_from_dict(M.stored(M.M1))) if s.optional}
    assert optional == {"l2.norm2", "l2.norm2.b", "l2.norm2.alpha", "l4.mix.vmix"}


@pytest.mark.parametrize("change, error", [
    (lambda c: c["layers"][0].update(type="conv"), UnsupportedError),
    (lambda c: c["layers"][0]["mixer"].update(gate_cap=0.0), InvalidArgumentError),
    (lambda c: c["layers"][0]["mixer"].pop("gate_cap"), InvalidArgumentError),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), InvalidArgumentError),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=5), InvalidArgumentError),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=32), InvalidArgumentError),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), InvalidArgumentError),
    (lambda c: c["layers"][2]["mixer"].pop("conv"), InvalidArgumentError),
    (lambda c: c["layers"][2]["mixer"].update(kv_heads=3), InvalidArgumentError),
    (lambda c: c["layers"][3]["mixer"].update(vdim=16), InvalidArgumentError),     # blends values of another shape
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), InvalidArgumentError),
    (lambda c: c["layers"][0]["mlp"].update(shared={}), InvalidArgumentError),
    (lambda c: c["layers"][1]["mlp"].update(kind="gated"), UnsupportedError),
    (lambda c: c.pop("norm"), InvalidArgumentError),
    (lambda c: c.pop("vocab"), InvalidArgumentError),
])
def test_a_bad_configuration_is_refused_with_its_key(change, error):
    data = copy.deepcopy(M.stored(M.M1))
    change(data)
    with pytest.raises(error):
        config_from_dict(data)


def test_the_command_line_reads_the_model(tmp_path, capsys):
    from vipera_rs_amd.cli import main

    folder = M.make_folder(tmp_path / "m2", M.M2, 1)
    assert main(["model-info", folder]) == 0
    out = capsys.readouterr().out
    assert "Muzasun" in out


# --- the plain implementation against closed forms of its own -------------------------------------------------------
def test_plain_matrix_memory_with_open_gates_is_a_normalized_running_sum():
    """Forget gates of one and input gates of one (both logarithms 0, so the running maximum stays 0): S is the plain sum
    of k v^T and the read-out S^T q / max(|sum k . q|, 1)."""
    rng = np.random.default_rng(1)
    T, W, H, D, V = 9, 12, 2, 4, 3
    h = rng.standard_normal((T, W))
    w = {"p.q": rng.standard_normal((H * D, W)), "p.k": rng.standard_normal((H * D, W)), "p.v": rng.standard_normal((H * V, W)),
         "p.i": np.zeros((H, W)), "p.i.b": np.zeros(H), "p.f": np.zeros((H, W)), "p.f.b": np.full(H, 1e9),
         "p.g": np.zeros((H * V, W)), "p.norm": np.ones(H * V), "p.o": np.eye(H * V)}
    got = P.matrix_memory_mixer(h, w, "p.", {"heads": H, "dim": D, "vdim": V, "gate_cap": 1e12}, 0.0)
    q = (h @ w["p.q"].T).reshape(T, H, D) / math.sqrt(D)
    k, v = (h @ w["p.k"].T).reshape(T, H, D), (h @ w["p.v"].T).reshape(T, H, V)
    want = np.zeros((T, H, V))
    for t in range(T):
        for head in range(H):
            top = sum(np.outer(k[s, head], v[s, head]) for s in range(t + 1)).T @ q[t, head]
            under = sum(k[s, head] for s in range(t + 1)) @ q[t, head]
            want[t, head] = top / (max(abs(under), 1.0) + 1e-6)
    want = P.over_rms(want, 0.0).reshape(T, H * V) * 0.5          # the gate is sigmoid(0)
    assert np.allclose(got, want, atol=1e-9)


def test_plain_delta_rule_without_decay_stores_and_overwrites():
    """One tap of 1 (the convolution passes its input through silu), decays of one, beta of one: writing value v under a
    unit key k and reading with the same key returns v; a second write under the same key replaces it."""
    D, V = 4, 3
    S = np.zeros((D, V))
    k = np.array([1.0, 0.0, 0.0, 0.0])
    for v in (np.array([1.0, 2.0, 3.0]), np.array([-1.0, 0.5, 4.0])):
        S = S + np.outer(k, 1.0 * (v - S.T @ k))
        assert np.allclose(S.T @ k, v)
    # and the mixer itself with a decay that halves one key channel only
    rng = np.random.default_rng(2)
    T, W, R = 6, 8, 2
    h = rng.standard_normal((T, W))
    m = {"heads": 1, "kv_heads": 1, "dim": D, "vdim": V, "conv": 1}
    w = {"p.q": rng.standard_normal((D, W)), "p.k": rng.standard_normal((D, W)), "p.v": rng.standard_normal((V, W)),
         "p.q.conv": np.ones((D, 1)), "p.k.conv": np.ones((D, 1)), "p.v.conv": np.ones((V, 1)),
         "p.b": np.zeros((1, W)), "p.A_log": np.zeros(1), "p.a1": np.zeros((R, W)), "p.a2": np.zeros((D, R)),
         "p.dt_bias": np.array([-1e9, -1e9, -1e9, math.log(math.e ** math.log(2.0) - 1.0)]),
         "p.g1": np.zeros((R, W)), "p.g2": np.zeros((V, R)), "p.norm": np.ones(V), "p.o": np.eye(V)}
    got = P.channel_delta_mixer(h, w, "p.", m, 0.0)
    q = P.silu(h @ w["p.q"].T)
    k = P.silu(h @ w["p.k"].T)
    v = P.silu(h @ w["p.v"].T)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) / math.sqrt(D)
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    S, want = np.zeros((D, V)), np.zeros((T, V))
    for t in range(T):
        S[3] *= 0.5                                   # softplus(dt_bias[3]) = log 2, exp(-exp(0) log 2) = 1/2
        S = S + np.outer(k[t], 0.5 * (v[t] - S.T @ k[t]))      # beta = sigmoid(0)
        want[t] = S.T @ q[t]
    assert np.allclose(got, P.over_rms(want, 0.0) * 0.5, atol=1e-9)


def test_plain_attention_rotation_depends_on_the_distance_only():
    rng = np.random.default_rng(3)
    x, y = rng.standard_normal((1, 1, 8)), rng.standard_normal((1, 1, 8))
    dots = [float((P.rotate_half(x, np.array([p + 5]), 4, 100.0) * P.rotate_half(y, np.array([p]), 4, 100.0)).sum())
            for p in (0, 3, 40)]
    assert np.allclose(dots, dots[0])
    turned = P.rotate_half(x, np.array([7]), 4, 100.0)
    assert np.array_equal(turned[..., 4:], x[..., 4:]) and not np.allclose(turned[..., :4], x[..., :4])
    # number i turns with number i + dims / 2
    one = np.zeros((1, 1, 8)); one[0, 0, 1] = 1.0
    angle = 7 * 100.0 ** (-2.0 / 4)
    want = np.zeros(8); want[1], want[3] = math.cos(angle), math.sin(angle)
    assert np.allclose(P.rotate_half(one, np.array([7]), 4, 100.0)[0, 0], want)


def test_plain_experts_weigh_their_inputs():
    rng = np.random.default_rng(4)
    W, F = 6, 5
    h = rng.standard_normal((3, W))
    w = {"p.router": rng.standard_normal((4, W))}
    for e in range(4):
        w[f"p.e{e}.gate"], w[f"p.e{e}.up"], w[f"p.e{e}.down"] = (rng.standard_normal(s) for s in ((F, W), (F, W), (W, F)))
    m = {"router": {"experts": 4, "top": 2}, "expert": {"ff": F}}
    got = P.mixture_of_experts(h, w, "p.", m)
    scores = P.sigmoid(h @ w["p.router"].T)
    for t in range(3):
        best = np.argsort(-scores[t])[:2]
        want = sum(w[f"p.e{e}.down"] @ (P.silu(w[f"p.e{e}.gate"] @ (scores[t, e] * h[t])) * (w[f"p.e{e}.up"] @ (scores[t, e] * h[t])))
                   for e in best)
        assert np.allclose(got[t], want)
    assert P.route(np.array([0.5, 0.7, 0.7, 0.1]), 2) == [1, 2] and P.route(np.array([0.7, 0.7, 0.7]), 1) == [0]
