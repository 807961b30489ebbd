"""Lurirax without a GPU: reading its configuration, the layer specs built from it, what a request keeps, declared
tensors against folders, refused configurations, and the plain implementation's mechanisms against closed forms."""
import copy
import json
import math
import os

import numpy as np
import pytest
import torch

import lurirax_helpers as L
import vipera_rs_amd  # noqa: F401
from plain import lurirax_plain as P
from vipera_rs_amd.config import LuriraxConfig, config_from_dict
from vipera_rs_amd.errors import InvalidArgumentError, UnsupportedError
from vipera_rs_amd.models import check_model, declare_cache_needs, declare_model
from vipera_rs_amd.parts.attention import distance_rows
from vipera_rs_amd.parts.rotary import neox_inverse_frequencies, stretch_long_waves


def test_the_registry_finds_the_configuration_by_its_name():
    cfg = config_from_dict(L.stored(L.L1))
    assert isinstance(cfg, LuriraxConfig) and cfg.vocab == 83 and cfg.width == 48 and cfg.embedding_scale == 1.5
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_layer_specs_carry_every_size_and_constant():
    specs = config_from_dict(L.L1).layer_specs()
    assert [s.block for s in specs] == ["postnorm"] * 4
    two, one, pair, last = (s.mixer for s in specs)
    assert two.kind == "attention" and two.params["maps"] == 2 and two.params["keep_first"] == 3
    assert two.params["window"] == 11 and two.params["qk_norm"] == "head" and two.params["diff"] == 0.4
    assert one.params["window"] == 9 and one.params["sink"] and one.params["qk_norm"] == "unit"
    assert specs[1].position.kind == "rotary_neox" and specs[1].position.params["rotary_dim"] == 8
    assert specs[1].position.params["long_waves"] == {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64.0}
    assert pair.kind == "mixer_pair" and pair.params["left_scale"] == 0.7 and pair.params["right_scale"] == 0.4
    left, right = pair.params["left"], pair.params["right"]
    assert left.params["chunk"] == 13 and left.params["gate"] == "head_sigmoid" and left.params["qkv_bias"]
    assert left.params["rel_bias"] == {"rows": 8, "far": 12.0} and left.params["sink"]
    assert right.kind == "decay_attention" and right.params["norm"] == "head" and right.params["k_scale"] == 0.25
    assert right.params["rotary"] == {"dims": 16, "base": 100.0} and right.params["gate"] == "silu"
    assert specs[0].ffn.kind == "gated_mlp" and specs[0].ffn.params["activation"] == "gelu_tanh"
    moe = specs[1].ffn.params
    assert (moe["experts"], moe["top"], moe["weight_scale"], moe["shared"], moe["scores"]) == (6, 2, 1.5, 16, "steered")
    assert config_from_dict(L.L2).layer_specs()[1].ffn.kind == "none"


def test_what_a_request_keeps():
    needs = declare_cache_needs(config_from_dict(L.L1))
    # kept first positions lie outside the window's bookkeeping: that layer keeps all its pages
    assert needs[0].kv.window == 0 and needs[0].kv.head_dim == 16 and needs[0].kv.kv_heads == 2 and needs[0].state is None
    assert needs[1].kv.window == 9 and needs[3].kv.window == 21
    assert needs[2].kv.window == 0 and needs[2].state is not None and needs[2].state.dtype == torch.float32
    wide = declare_cache_needs(config_from_dict(L.L2))
    assert wide[0].kv.head_dim == 32 and wide[1].kv.head_dim == 32      # max(dim, vdim) and two maps side by side


def test_declared_tensors_match_a_folder(tmp_path):
    from vipera_rs_amd.weights import Checkpoint

    for name, cfg in (("l1", L.L1), ("l2", L.L2)):
        folder = L.make_folder(tmp_path / name, cfg, 3)
        with open(os.path.join(folder, "config.json")) as handle:
            stored = json.load(handle)
        assert "bias_rows" not in json.dumps(stored)              # the table's rows are the tensor's own
        specs = declare_model(config_from_dict(stored))
        checkpoint = Checkpoint(folder)
        try:
            checkpoint.check(specs)
            assert {s.name for s in specs if not s.optional} <= set(checkpoint.names())
        finally:
            checkpoint.close()
        check_model(config_from_dict(stored), torch.bfloat16)


def test_refused_configurations():
    def broken(change):
        cfg = copy.deepcopy(L.L1)
        change(cfg)
        return cfg

    with pytest.raises(UnsupportedError):
        config_from_dict(broken(lambda c: c["layers"][0].update(type="attention_3")))
    with pytest.raises(InvalidArgumentError):
        config_from_dict(broken(lambda c: c["layers"][1]["mixer"].update(kv_heads=3)))
    with pytest.raises(InvalidArgumentError):
        config_from_dict(broken(lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7)))
    with pytest.raises(InvalidArgumentError):
        config_from_dict(broken(lambda c: c["layers"][2]["mixer"]["right"].update(decay=[0.5])))
    with pytest.raises(InvalidArgumentError):
        config_from_dict(broken(lambda c: c["layers"][1]["mlp"]["router"].update(top=9)))
    with pytest.raises(InvalidArgumentError):
        config_from_dict(broken(lambda c: c["layers"][0]["mixer"].pop("diff")))
    with pytest.raises(UnsupportedError):
        config_from_dict(broken(lambda c: c["layers"][3].update(mlp={"kind": "sparse"})))


# --- the plain mechanisms against closed forms of their own ---------------------------------------------------------
def test_rows_of_the_table_by_distance():
    assert [P.distance_bucket(n, 8, 40) for n in range(4)] == [0, 1, 2, 3]
    assert P.distance_bucket(4, 8, 40) == 4 and P.distance_bucket(39, 8, 40) == 7 and P.distance_bucket(4000, 8, 40) == 7
    # logarithmic steps: the first distance of row 4 + j is the first n with (n / 4) >= 10^(j / 4)
    edges = [min(n for n in range(4, 41) if P.distance_bucket(n, 8, 40) == row) for row in range(4, 8)]
    assert edges == [4, 8, 13, 23]
    for rows, far in ((8, 40), (6, 9.5), (16, 200), (2, 3)):
        assert distance_rows(rows, far, 300) == [P.distance_bucket(n, rows, far) for n in range(301)]


def test_long_waves_are_stretched():
    rot = {"dims": 16, "base": 500.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}
    plain = P.frequencies(rot)
    base = 500.0 ** (-np.arange(8) / 8.0)
    wave = 2 * math.pi / base
    assert np.allclose(plain[wave < 16], base[wave < 16]) and np.allclose(plain[wave > 64], base[wave > 64] / 4.0)
    between = (wave >= 16) & (wave <= 64)
    assert between.any() and np.all(plain[between] < base[between]) and np.all(plain[between] > base[between] / 4.0)
    table = stretch_long_waves(neox_inverse_frequencies(16, 500.0), 4.0, 1.0, 4.0, 64)
    assert np.allclose(table, plain, rtol=1e-6)


def test_rotation_enters_scores_by_distance_only():
    rng = np.random.default_rng(1)
    q, k = rng.standard_normal((1, 1, 12)), rng.standard_normal((1, 1, 12))
    rot = {"dims": 8, "base": 100.0}
    dots = [float(np.sum(P.rotate(q, [a], rot) * P.rotate(k, [a - 5], rot))) for a in (5, 9, 300)]
    assert np.allclose(dots, dots[0]) and not np.isclose(dots[0], float(np.sum(q * k)))
    assert np.allclose(P.rotate(q, [7], rot)[..., 8:], q[..., 8:])           # the rest passes unchanged


def test_a_sink_takes_its_share_and_adds_nothing():
    rng = np.random.default_rng(2)
    q, k, v = rng.standard_normal((5, 2, 4)), rng.standard_normal((5, 1, 4)), rng.standard_normal((5, 1, 3))
    mask = P.visible("full", 0, 0, 5)
    plain = P.softmax_attention(q, k, v, 0.5, mask)
    far_down = P.softmax_attention(q, k, v, 0.5, mask, sink=np.array([-80.0, -80.0]))
    assert np.allclose(plain, far_down)
    sink = np.array([0.3, 50.0])
    out = P.softmax_attention(q, k, v, 0.5, mask, sink=sink)
    s = q[4, 0] @ k[:, 0].T * 0.5
    share = np.exp(s).sum() / (np.exp(s).sum() + math.exp(0.3))
    assert np.allclose(out[4, 0], plain[4, 0] * share) and np.allclose(out[:, 1], 0.0, atol=1e-12)


def test_masks():
    w = P.visible("window", 3, 2, 9)
    assert [j for j in range(9) if w[8, j]] == [0, 1, 6, 7, 8] and [j for j in range(9) if w[3, j]] == [0, 1, 2, 3]
    c = P.visible("chunk", 4, 0, 9)
    assert [j for j in range(9) if c[6, j]] == [4, 5, 6] and [j for j in range(9) if c[8, j]] == [8]


def test_retention_is_a_decayed_sum_of_outer_products():
    cfg = L.single(L.parallel(L.chunked(1, 1, 4, 4, 5), L.retention(1, 4, 3, decay=[0.5], rot_dims=0)), width=8)
    w = {k: t.double().numpy() for k, t in L.make_weights(cfg, 1).items()}
    x = np.random.default_rng(3).standard_normal((6, 8))
    m, pre = cfg["layers"][0]["mixer"]["right"], "l0.mix.right."
    q, k, v = x @ w[pre + "q"].T, x @ w[pre + "k"].T * 0.5, x @ w[pre + "v"].T
    o = np.stack([sum(0.5 ** (t - s) * (q[t] @ k[s]) * v[s] for s in range(t + 1)) for t in range(6)])
    want = (P.over_rms(o, 1e-5) * P.silu(x @ w[pre + "g"].T)) @ w[pre + "o"].T
    assert np.allclose(P.retention(x, w, pre, m, 1e-5), want)


def test_experts_are_chosen_with_the_correction_and_weighed_without():
    cfg = L.single(L.windowed(1, 1, 4, 4, 3), L.moe(4, 2, 6, scale=2.0), width=8)
    w = {k: t.double().numpy() for k, t in L.make_weights(cfg, 2).items()}
    pre = "l0.mlp."
    w[pre + "router"] = np.zeros((4, 8))
    w[pre + "router"][:, 0] = [3.0, 2.0, 1.0, 0.0]
    w[pre + "correction"] = np.array([0.0, -1.0, 0.0, 1.0])
    x = np.zeros((1, 8))
    x[0, 0] = 1.0
    x[0, 1:] = 0.3
    s = P.sigmoid(np.array([3.0, 2.0, 1.0, 0.0]))
    assert P.choose(list(s + w[pre + "correction"]), 2) == [3, 0]             # expert 3 only through its correction
    expert = lambda e: P.gated_feed_forward(x, w, f"{pre}e{e}.", P.silu)
    want = 2.0 * (s[3] * expert(3) + s[0] * expert(0))
    assert np.allclose(P.mixture_of_experts(x, w, pre, cfg["layers"][0]["mlp"]), want)
    assert P.choose([0.5, 0.7, 0.7, 0.1], 2) == [1, 2] and P.choose([0.2, 0.2, 0.2], 1) == [0]


def test_two_maps_with_equal_weights_cancel_to_the_difference_of_lambda():
    """With both maps equal, a_1 = a_2 and the head's output is (1 - lambda) a, normed: its direction is a's."""
    cfg = L.single(L.differential(1, 1, 4, 6, 50, keep_first=0, diff=0.25), width=8)
    w = {k: t.double().numpy() for k, t in L.make_weights(cfg, 4).items()}
    pre = "l0.mix."
    w[pre + "q"][4:] = w[pre + "q"][:4]
    w[pre + "k"][4:] = w[pre + "k"][:4]
    w[pre + "o"] = np.eye(8)[:, :6]
    x = np.random.default_rng(5).standard_normal((7, 8))
    out = P.differential_attention(x, w, pre, cfg["layers"][0]["mixer"], 1e-6)[:, :6]
    q = P.over_rms((x @ w[pre + "q"].T).reshape(7, 1, 2, 4), 1e-6)[:, :, 0] * w[pre + "q.norm"]
    k = P.over_rms((x @ w[pre + "k"].T).reshape(7, 1, 2, 4), 1e-6)[:, :, 0] * w[pre + "k.norm"]
    a = P.softmax_attention(q, k, (x @ w[pre + "v"].T).reshape(7, 1, 6), cfg["layers"][0]["mixer"]["scale"],
                            P.visible("full", 0, 0, 7))[:, 0]
    lam = math.exp(float(w[pre + "lq1"] @ w[pre + "lk1"])) - math.exp(float(w[pre + "lq2"] @ w[pre + "lk2"])) + 0.25
    assert np.allclose(out, np.sign(1 - lam) * P.over_rms(a, 1e-6) * 0.75, atol=1e-5)


def test_model_info_names_the_architecture(tmp_path):
    import subprocess
    import sys

    folder = L.make_folder(tmp_path / "l2", L.L2, 5)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "vipera"), "model-info", folder], capture_output=True,
                          text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert "Lurirax" in done.stdout
