"""Rukosun without a GPU: the configuration reader, the model it describes, the tensors it declares, and the plain
implementation's mechanisms against hand-made cases."""
import copy

import numpy as np
import pytest

from tests import rukosun_helpers as RH
from tests.plain import rukosun_plain as R


def test_registry_and_run_order():
    from gibbs_amd.config import RukosunConfig, config_from_dict
    cfg = config_from_dict(RH.RUKOSUN_P)
    assert isinstance(cfg, RukosunConfig)
    spec = cfg.model_spec()
    assert spec.order == (0, 1, 2, 1, 2, 1, 2, 3) and spec.streams == 2 and spec.max_position == 400
    assert spec.embedding_tables.buckets == 97 and spec.embedding_tables.positions == 400
    assert config_from_dict(RH.RUKOSUN_R).model_spec().order == (0, 1, 2)
    assert R.run_order(RH.RUKOSUN_P) == list(spec.order) and R.run_order(RH.RUKOSUN_Q) == [0, 1, 2, 0, 1, 2]
    assert cfg.to_dict() == RH.RUKOSUN_P and cfg.derived()["order"] == list(spec.order)


def test_mixers_constants_come_from_the_configuration():
    from gibbs_amd.config import config_from_dict
    spec = config_from_dict(RH.RUKOSUN_P).model_spec()
    first, second = spec.layers[0].part("mixer"), spec.layers[1].part("mixer")
    assert first.params["q_rank"] == 30 and first.params["sink"] and first.params["gate"] and first.params["window"] == 5
    assert first.position.params == {"theta": 1000.0, "rotary_dim": 6, "variant": "interleaved", "precision": "f64"}
    assert second.params["q_rank"] is None and not second.params["sink"] and not second.params["gate"]
    assert second.position.params["variant"] == "half_split" and second.position.params["theta"] == 300.0
    assert spec.layers[2].part("mixer").params["window"] is None
    assert [r for r, _ in spec.layers[1].parts] == ["norm1", "mixer", "connection1"]
    assert [r for r, _ in spec.layers[0].parts] == ["norm1", "mixer", "connection1", "norm2", "ffn", "connection2"]
    plain = config_from_dict(RH.RUKOSUN_R).model_spec()
    assert plain.streams == 1 and [r for r, _ in plain.layers[0].parts] == ["norm1", "mixer", "norm2", "ffn"]
    assert plain.embedding_tables.pair is None and plain.embedding_tables.position == "pos"


def test_declared_tensors():
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    model = DecoderModel(config_from_dict(RH.RUKOSUN_P).model_spec())
    shapes = {d.name: d.shape for d in model.tensor_decls()}
    assert shapes["bigram"] == (98, 100) and shapes["pos"] == (400, 100) and shapes["final.norm.b"] == (100,)
    assert shapes["l0.mix.dq"] == (30, 100) and shapes["l0.mix.uq"] == (3 * 18, 30) and shapes["l0.mix.dkv"] == (27, 100)
    assert shapes["l0.mix.uk"] == (36, 21) and shapes["l0.mix.uv"] == (60, 21) and shapes["l0.mix.sink"] == (3,)
    assert shapes["l0.mix.g"] == (60, 100) and shapes["l0.mix.o"] == (100, 60) and shapes["l0.mlp.act"] == (4,)
    assert shapes["l1.mix.q"] == (70, 100) and "l1.mix.sink" not in shapes and "l1.mix.g" not in shapes and "l1.norm2" not in shapes
    assert shapes["l0.hc1.mix"] == (2, 2) and shapes["l0.hc2.in"] == (2,) and "l1.hc2.in" not in shapes
    need = model.cache_needs()
    assert need[0].kv_heads == 1 and need[0].head_dim == 27 and need[0].window == 5 and need[0].value_dim == 0
    assert need[-1] is None and model.state_needs()[-1][0].dtype == "int32" and model.model_state_owner() == 8
    assert len(need) == 9 and need[2].window is None


def test_a_second_norm_without_a_feed_forward_is_accounted_for():
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights.loader import check_table
    model = DecoderModel(config_from_dict(RH.RUKOSUN_P).model_spec())
    table = {d.name: d.shape for d in model.tensor_decls()}
    table.update({"l1.norm2": (100,), "l1.norm2.b": (100,), "l1.hc2.in": (2,), "l1.hc2.out": (2,), "l1.hc2.mix": (2, 2)})
    again = DecoderModel(config_from_dict(RH.RUKOSUN_P, tensors=table).model_spec())
    check_table(again.tensor_decls(), table)


@pytest.mark.parametrize("key", ["width", "vocab", "norm", "max_positions", "layers"])
def test_missing_keys_are_named(key):
    from gibbs_amd.config import ConfigError, config_from_dict
    cfg = copy.deepcopy(RH.RUKOSUN_R)
    del cfg[key]
    with pytest.raises(ConfigError, match=key if key != "norm" else "norm.eps"):
        config_from_dict(cfg)


def test_bad_values_are_refused():
    from gibbs_amd.config import ConfigError, config_from_dict
    for change in (lambda c: c["layers"][0].update(type="attention"), lambda c: c["layers"][1]["mixer"].pop("q_rank"),
                   lambda c: c.update(streams=9), lambda c: c.update(loop={"start": 2, "stop": 1, "times": 2}),
                   lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), lambda c: c["layers"][0]["mlp"].update(kind="experts")):
        cfg = copy.deepcopy(RH.RUKOSUN_R)
        change(cfg)
        with pytest.raises(ConfigError):
            config_from_dict(cfg)


# ----------------------------------------------------------------------------------------------- the plain mechanisms
def test_plain_pair_rows_and_first_token():
    rows = R.bigram_rows([5, 9, 9, 0], 13, 3, 4)
    assert rows.tolist() == [13, (5 * 3 + 9 * 4) % 13, (9 * 3 + 9 * 4) % 13, (9 * 3) % 13]


def test_plain_rotation_pairs():
    x = np.arange(8, dtype=np.float64)[None, None, :] + 1.0
    inter = R.rotate(x, [3], 100.0, 4, True)[0, 0]
    half = R.rotate(x, [3], 100.0, 4, False)[0, 0]
    f = np.array([1.0, 100.0 ** -0.5])
    c, s = np.cos(3 * f), np.sin(3 * f)
    assert np.allclose(inter[:4], [1 * c[0] - 2 * s[0], 2 * c[0] + 1 * s[0], 3 * c[1] - 4 * s[1], 4 * c[1] + 3 * s[1]], atol=1e-6)
    assert np.allclose(half[:4], [1 * c[0] - 3 * s[0], 2 * c[1] - 4 * s[1], 3 * c[0] + 1 * s[0], 4 * c[1] + 2 * s[1]], atol=1e-6)
    assert np.array_equal(inter[4:], x[0, 0, 4:]) and np.array_equal(half[4:], x[0, 0, 4:])


def test_plain_window_and_sink():
    T = 6
    q = np.zeros((T, 1, 2)); k = np.zeros((T, 1, 2)); v = np.eye(T)[:, None, :]
    out = R.windowed_softmax_attention(q, k, v, 1.0, 3)          # equal scores: the mean of what is seen
    assert np.allclose(out[5, 0], [0, 0, 0, 1 / 3, 1 / 3, 1 / 3]) and np.allclose(out[1, 0], [.5, .5, 0, 0, 0, 0])
    out = R.windowed_softmax_attention(q, k, v, 1.0, 3, sink=np.array([np.log(3.0)]))   # the sink weighs as three keys
    assert np.allclose(out[5, 0], [0, 0, 0, 1 / 6, 1 / 6, 1 / 6]) and np.allclose(out[0, 0], [1 / 4, 0, 0, 0, 0, 0])
    assert np.allclose(R.windowed_softmax_attention(q, k, v, 1.0, None)[5, 0], np.full(T, 1 / 6))


def test_plain_poly_norm_and_hyper_connection():
    z = np.array([[1.0, -2.0, 3.0, 0.5]])
    n = lambda a: a / np.sqrt((a * a).mean() + 1e-6)
    assert np.allclose(R.poly_norm(z, [0.5, -1.0, 2.0, 0.25], 1e-6), 0.5 * n(z) - n(z ** 2) + 2 * n(z ** 3) + 0.25)
    xs = np.stack([np.full((2, 3), 1.0), np.full((2, 3), 10.0)])
    mix = np.array([[1.0, 2.0], [3.0, 4.0]])                      # [from, to]
    new = R.hyper_write(xs, mix, np.array([5.0, 7.0]), np.full((2, 3), 100.0))
    assert np.allclose(new[0], 1 * 1 + 3 * 10 + 500) and np.allclose(new[1], 2 * 1 + 4 * 10 + 700)
    assert np.allclose(R.hyper_read(xs, np.array([2.0, 0.5])), 7.0)
