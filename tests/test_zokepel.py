"""Zokepel without a GPU: its configuration, the order of its runs, the distance buckets, the tensors it declares,
and the plain implementation's mechanisms against properties that follow from their equations."""
import json
import math

import numpy as np
import pytest

from tests import zokepel_helpers as ZH
from tests.plain import zokepel_plain as Z


def test_registry_finds_the_architecture_by_its_key():
    from gibbs_amd.config import ZokepelConfig, config_from_dict
    cfg = config_from_dict(ZH.ZOKEPEL_P)
    assert isinstance(cfg, ZokepelConfig)
    assert config_from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg


@pytest.mark.parametrize("loop,order,again", [
    (None, (0, 1, 2, 3), ()),
    ({"start": 1, "stop": 3, "times": 3}, (0, 1, 2, 1, 2, 1, 2, 3), (3, 5)),
    ({"start": 0, "stop": 4, "times": 2}, (0, 1, 2, 3, 0, 1, 2, 3), (4,)),
    ({"start": 2, "stop": 4, "times": 1}, (0, 1, 2, 3), ()),
    ({"start": 2, "stop": 2, "times": 5}, (0, 1, 2, 3), ()),
])
def test_run_order(loop, order, again):
    from gibbs_amd.config import config_from_dict
    cfg = dict(ZH.ZOKEPEL_P, loop=loop)
    if loop is None:
        del cfg["loop"]
    spec = config_from_dict(cfg).model_spec()
    assert spec.order == order and spec.reinject_before == again
    plain = Z.run_order(cfg)
    assert tuple(i for i, _ in plain) == order and tuple(n for n, (_, a) in enumerate(plain) if a) == again


def test_sizes_that_only_tensor_shapes_give():
    from gibbs_amd.config import ConfigError, config_from_dict
    from gibbs_amd.parts import DecoderModel
    cfg = json.loads(json.dumps(ZH.ZOKEPEL_P))
    table = {d.name: d.shape for d in DecoderModel(config_from_dict(cfg).model_spec()).tensor_decls()}
    for layer in cfg["layers"]:                     # a config.json as a checkpoint brings it: without those keys
        m = layer["mixer"]
        for section in (m, m.get("left", {}), m.get("right", {})):
            for key in ("bias_rows", "decay_rank", "gate_rank"):
                section.pop(key, None)
    with pytest.raises(ConfigError):
        config_from_dict(cfg)
    spec = config_from_dict(cfg, tensors=table).model_spec()
    assert {d.name: d.shape for d in DecoderModel(spec).tensor_decls()} == table
    assert "l1.norm2" not in table and "l1.mlp.gate" not in table          # the layer without a feed-forward
    table["l1.norm2"] = (cfg["width"],)                                     # a checkpoint that holds the norm all the same
    assert "l1.norm2" in {d.name for d in DecoderModel(config_from_dict(cfg, tensors=table).model_spec()).tensor_decls()}


def test_bad_configurations_are_refused():
    from gibbs_amd.config import ConfigError, config_from_dict
    for change in ({"layers": []}, {"loop": {"start": 3, "stop": 2, "times": 2}}, {"loop": {"start": 0, "stop": 9, "times": 2}},
                   {"norm": {}}, {"embedding": {}}):
        with pytest.raises(ConfigError):
            config_from_dict(dict(ZH.ZOKEPEL_P, **change))
    bad = json.loads(json.dumps(ZH.ZOKEPEL_P))
    bad["layers"][0]["type"] = "window"
    with pytest.raises(ConfigError):
        config_from_dict(bad)


@pytest.mark.parametrize("rows,reach", [(12, 50), (8, 40), (9, 30), (16, 128), (32, 1000)])
def test_distance_buckets(rows, reach):
    from gibbs_amd.parts.distance_bias import distance_buckets
    mine = distance_buckets(rows, reach)
    assert len(mine) == reach + 1 and mine == [Z.distance_bucket(n, rows, reach) for n in range(reach + 1)]
    assert mine[:rows // 2] == list(range(rows // 2)) and mine[-1] == rows - 1
    assert all(b >= a for a, b in zip(mine, mine[1:])) and max(mine) == rows - 1
    assert all(Z.distance_bucket(n, rows, reach) == rows - 1 for n in (reach, reach + 1, 10 * reach))


def test_random_model_folder_runs_through_the_plain_implementation(tmp_path):
    d = ZH.make_model_dir(str(tmp_path), ZH.ZOKEPEL_R, "R")
    logits = ZH.plain_logits(d, ZH.tokens(0, 19, 97))
    assert logits.shape == (19, 97) and np.isfinite(logits).all()
    # causal: a later token changes nothing before it
    other = ZH.plain_logits(d, ZH.tokens(0, 19, 97)[:11] + [5])
    assert np.allclose(other[:11], logits[:11], atol=1e-12)


def test_plain_delta_rule_recalls_what_it_wrote():
    rng = np.random.default_rng(0)
    D, V, T = 8, 5, 8
    keys = np.linalg.qr(rng.normal(size=(D, D)))[0]            # orthonormal keys: every write lands in its own direction
    values = rng.normal(size=(T, V))
    ones = np.ones(T)
    out = Z.delta_rule(keys, keys, values, ones, ones)         # beta 1, no decay: reading with a key right after its write
    assert np.allclose(out, values)
    # reading the first key again at the end, after 7 more writes and with a decay of 0.9 a token
    q = np.tile(keys[0], (T, 1))
    out = Z.delta_rule(q, keys, values, ones, np.full(T, 0.9))
    assert np.allclose(out[-1], values[0] * 0.9 ** 7)
    # a decay per key channel acts on the rows of the state
    g = np.ones((T, D)); g[1:, 0] = 0.5
    e = np.eye(D)
    out = Z.delta_rule(np.tile(e[0], (T, 1)), e, values, ones, g)
    assert np.allclose(out[-1], values[0] * 0.5 ** 7)


def test_plain_time_mix_state_is_a_decayed_sum():
    rng = np.random.default_rng(1)
    T, W, H, D, R = 6, 10, 2, 3, 4
    w = {n: rng.normal(size=s) * 0.5 for n, s in {"r": (H * D, W), "k": (H * D, W), "v": (H * D, W), "g": (H * D, W), "w1": (R, W),
                                                   "w2": (H * D, R), "w0": (H * D,), "u": (H, D), "norm": (H * D,), "o": (W, H * D)}.items()}
    w.update({"mu." + s: rng.uniform(size=W) for s in "rkvgw"})
    h = rng.normal(size=(T, W))
    got = Z.time_mix(h, w, {"heads": H, "dim": D}, 1e-5)
    # the same from the closed form: o_t = sum_{s<t} (prod_{s<m<t} w_m) k_s v_s^T r_t + u k_t v_t^T r_t
    prev = np.vstack([np.zeros((1, W)), h[:-1]])
    mix = lambda s: h + (prev - h) * w["mu." + s]
    r, k, v = ((mix(s) @ w[s].T).reshape(T, H, D) for s in "rkv")
    decay = np.exp(-np.exp(np.tanh(mix("w") @ w["w1"].T) @ w["w2"].T + w["w0"])).reshape(T, H, D)
    out = np.zeros((T, H, D))
    for t in range(T):
        for head in range(H):
            acc = w["u"][head] * k[t, head] * (r[t, head])
            total = np.outer(acc, v[t, head]).sum(0)
            for s in range(t):
                keep = np.prod(decay[s + 1:t, head], axis=0) if t - s > 1 else np.ones(D)
                total += (keep * k[s, head] * r[t, head]).sum() * v[s, head]
            out[t, head] = total
    want = (Z.unit_rms(out, 1e-5).reshape(T, H * D) * w["norm"] * Z.silu(mix("g") @ w["g"].T)) @ w["o"].T
    assert np.allclose(got, want)


def test_plain_conv_and_feed_forward():
    x = np.arange(12, dtype=float).reshape(6, 2)
    taps = np.array([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]])
    y = Z.causal_conv(x, taps)
    assert np.allclose(y[:, 1], x[:, 1]) and y[0, 0] == 0 and y[1, 0] == 200 + 0 and y[2, 0] == 400 + 20 + 0
    h = np.array([[1.0, -2.0]])
    eye = np.eye(2)
    big = Z.clamped_glu(h * 10, eye, eye, eye, 1.5)            # gate 10 -> 1.5; up -20 -> -1.5, then gate * sigmoid(1.702 gate) * (1 + up)
    assert np.allclose(big[0, 0], 1.5 * Z.sigmoid(1.702 * 1.5) * 2.5)
    assert np.allclose(big[0, 1], -20 * Z.sigmoid(1.702 * -20) * (-0.5))    # the gate is clamped from above only
    assert math.isclose(Z.sinusoid([3], 4)[0, 1], math.cos(3.0), rel_tol=1e-6) and Z.sinusoid([0], 6)[0].tolist() == [0, 1, 0, 1, 0, 1]
