"""The plain implementation of the Gulidra decoder pinned by values worked out by hand, and what needs no GPU of the
design's place in the framework: configuration, tensor names, cache needs."""
import math

import numpy as np
import pytest

import plain_gulidra as P
from gulidra_helpers import CONFIGS, TINY_GA, model_folder, oracle, tokens_for


def test_embedding_scales_the_token_row_only():
    table, pos = np.array([[1.0, 2.0], [3.0, 4.0]]), np.array([[10.0, 20.0], [30.0, 40.0], [50.0, 60.0]])
    assert np.array_equal(P.embed(table, pos, [1, 0], 1, 2.0), [[36.0, 48.0], [52.0, 64.0]])


def test_linear_attention_by_hand():
    """One head, keys and values of size 1: S_t = d S_(t-1) + k_t v_t, o_t = S_t q_t."""
    q, k, v = np.array([1.0, 2.0, 3.0]), np.array([1.0, 1.0, 2.0]), np.array([2.0, 4.0, 1.0])
    o, S = P.decayed_linear_attention(q.reshape(3, 1, 1), k.reshape(3, 1, 1), v.reshape(3, 1, 1), np.array([0.5]))
    assert np.allclose(o.ravel(), [2.0, 2 * (0.5 * 2 + 4), 3 * (0.5 * 5 + 2)]) and np.allclose(S, 4.5)
    o2, S2 = P.decayed_linear_attention(q[2:].reshape(1, 1, 1), k[2:].reshape(1, 1, 1), v[2:].reshape(1, 1, 1),
                                        np.array([0.5]), state=np.array([[[5.0]]]))
    assert np.allclose(o2, o[2]) and np.allclose(S2, S)


def test_differential_combination_by_hand():
    """Two keys; map 1 looks at the last key only, map 2 at both alike: a1 = v_1, a2 = (v_0 + v_1) / 2."""
    big = 50.0
    q = np.zeros((1, 1, 2, 2))
    q[0, 0, 0] = [big, 0.0]
    k = np.zeros((2, 1, 2, 2))
    k[1, 0, 0] = [1.0, 0.0]
    v = np.array([[[1.0, 3.0]], [[5.0, -1.0]]])
    lam, diff = 0.5, 0.2
    got = P.differential_attention(q, k, v, 1.0, lam, diff, 0.0)[0, 0]
    o = v[1, 0] - lam * (v[0, 0] + v[1, 0]) / 2
    assert np.allclose(got, o / math.sqrt(np.mean(o * o)) * 0.8)
    assert math.isclose(P.diff_lambda([1.0, 0.0], [2.0, 5.0], [0.5, 0.5], [1.0, 1.0], 0.3), math.exp(2) - math.exp(1) + 0.3)


def test_router_by_hand():
    """Three experts and one identity, two chosen: the correction moves the choice, the weights stay softmax scores."""
    h = np.array([[1.0, 0.0]])
    wr = np.array([[math.log(4.0), 0], [math.log(2.0), 0], [0.0, 0], [0.0, 0]])       # scores 4/8, 2/8, 1/8, 1/8
    ids, w = P.route(h, wr, np.zeros(4), 2)
    assert ids.tolist() == [[0, 1]] and np.allclose(w, [[0.5, 0.25]])
    ids, w = P.route(h, wr, np.array([0.0, 0.0, 0.0, 0.2]), 2)
    assert ids.tolist() == [[0, 3]] and np.allclose(w, [[0.5, 0.125]])
    ex = [(np.eye(2), np.eye(2), 2 * np.eye(2))] * 3
    out = P.routed_experts(h, wr, np.array([0.0, 0.0, 0.0, 0.2]), ex, 1, 2)
    unit = 2 * P.silu(h) * h
    assert np.allclose(out, 0.5 * unit + 0.125 * h)      # the identity expert returns its input, times its score


def test_prefill_equals_decoding_in_the_plain_model():
    for name in CONFIGS:
        m = oracle(model_folder(name))
        toks = tokens_for(name, 30, 4)
        mem = m.new_memory()
        parts = np.concatenate([m.forward(toks[:11], mem), m.forward(toks[11:13], mem)] +
                               [m.forward([t], mem) for t in toks[13:]])
        assert np.abs(parts - m.forward(toks)).max() < 1e-10


def test_configuration_and_tensor_names():
    from allpaca_amd.config import ConfigError
    from allpaca_amd.models import DecoderModel, describe_model
    arch, cfg, spec = describe_model(TINY_GA)
    assert arch.name == "gulidra" and cfg.residual_mult == 0.7 and cfg.layers[1].mixer.kv_from == 0
    names = DecoderModel(spec).param_specs()
    assert names["l1.mix.q"].shape == (4 * 2 * 12, 36) and "l1.mix.k" not in names and "l1.mix.k.norm" not in names
    assert names["l0.mix.k"].shape == (2 * 2 * 12, 36) and names["l0.mix.g"].shape == (4, 36)
    assert names["l0.mix.q.conv"].shape == (96, 3) and names["l1.mix.q.conv"].shape == (96, 2)
    assert "l4.mix.q.conv" not in names and names["l4.mix.lq2"].shape == (10,)
    assert names["l2.mix.g"].shape == (24, 36) and names["l2.mix.norm"].shape == (24,) and "l2.norm2" not in names
    assert names["l1.mlp.router"].shape == (7, 36) and names["l1.mlp.correction"].shape == (7,)
    assert "l1.mlp.e4.down" in names and "l1.mlp.e5.down" not in names and names["pos"].shape == (300, 36)
    for change, text in [(dict(residual_mult=None), "residual_mult"), (dict(embedding={}), "scale"),
                         (dict(max_positions=0), "max_positions")]:
        with pytest.raises(ConfigError, match=text):
            describe_model({**TINY_GA, **change})
    bad = dict(TINY_GA, layers=[dict(TINY_GA["layers"][2], mixer=dict(TINY_GA["layers"][2]["mixer"], decay=[0.5]))])
    with pytest.raises(ConfigError, match="decay"):
        describe_model(bad)
    bad = dict(TINY_GA, layers=[TINY_GA["layers"][2], TINY_GA["layers"][1]])       # keys of a layer that has none
    with pytest.raises(ConfigError, match="kv_from"):
        describe_model(bad)


def test_cache_needs_of_owners_borrowers_and_recurrent_layers():
    from allpaca_amd.models import DecoderModel, describe_model
    from allpaca_amd.parts import FixedState, PagedKeysValues
    _, _, spec = describe_model(TINY_GA)
    needs = DecoderModel(spec).cache_needs()
    assert needs[0] == {"mixer": PagedKeysValues(2, 24, 20), "mixer.state": FixedState((2, 4 * 24 + 2 * (24 + 20)))}
    assert needs[1] == {"mixer.state": FixedState((1, 4 * 24))}        # borrowed pages, its own rows for its own taps
    assert needs[2] == FixedState((2, 20, 12)) and needs[3] == FixedState((3, 6, 28))
    assert needs[4] == PagedKeysValues(2, 20, 6)                        # no convolution: nothing but pages
    assert spec.plan[1].cache_of == 0 and spec.plan[2].cache_of is None
