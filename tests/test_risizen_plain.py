"""The Risizen decoder without a GPU: the configuration reader, the description in parts, tensor names, what each
plan entry asks of the cache manager, and the plain implementation's own mechanisms against each other (it is the
yardstick of the GPU tests, so its pieces are pinned here with numbers worked out by hand or in a second way)."""
import copy

import numpy as np
import pytest
import torch

import plain_risizen as R
from risizen_helpers import CONFIGS, TINY_RA, TINY_RB, TINY_RD, model_folder, oracle, tokens_for

from allpaca_amd.config import ConfigError
from allpaca_amd.models import DecoderModel, describe_model
from allpaca_amd.parts import PagedKeysValues


# ------------------------------------------------------------------------------------------- the plain mechanisms
def test_short_conv_by_hand_and_with_rows_ahead():
    u = np.array([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0], [4.0, 40.0]])
    w = np.array([[0.5, 1.0, 2.0], [1.0, 0.0, -1.0]])           # [channels, taps]: the last tap is the row itself
    y = R.short_conv(u, w)
    assert np.allclose(y[:, 0], [2.0, 5.0, 8.5, 12.0])            # 2*1 | 1*1+2*2 | .5*1+1*2+2*3 | .5*2+1*3+2*4
    assert np.allclose(y[:, 1], [-10.0, -20.0, -20.0, -20.0])
    # cutting the rows anywhere and handing over the last two gives the same
    for cut in (1, 2, 3):
        ext = np.concatenate([np.zeros((2, 2)), u[:cut]])
        assert np.allclose(R.short_conv(u[cut:], w, before=ext[-2:]), y[cut:])


def test_mask_edges():
    assert R.visible(6, 0, 7) and R.visible(6, 6, 7) and not R.visible(6, 7, 7)
    assert not R.visible(7, 6, 7) and R.visible(7, 7, 7) and R.visible(13, 7, 7) and not R.visible(14, 13, 7)
    assert R.visible(100, 0, None) and not R.visible(3, 4, None)


def test_sink_takes_its_share():
    q = np.zeros((1, 1, 4))                                        # every score is 0, like the sink's
    k, v = np.ones((3, 1, 4)), np.array([[[1.0]], [[2.0]], [[6.0]]])
    assert np.allclose(R.sink_attention(q, k, v, 1.0, None), [[9.0 / 4.0]])       # (1 + 2 + 6) / (1 + 3)
    assert np.allclose(R.sink_attention(q, k, v, 1.0, None, sink=False), [[3.0]])
    # large scores: the sink's share vanishes
    q[0, 0] = 50.0
    assert np.allclose(R.sink_attention(q, k, v, 1.0, None), [[3.0]])


def test_grouped_heads_and_chunks_in_attention():
    rng = np.random.default_rng(0)
    q, k, v = rng.normal(size=(9, 4, 6)), rng.normal(size=(9, 2, 6)), rng.normal(size=(9, 2, 3))
    out = R.sink_attention(q, k, v, 0.7, 4).reshape(9, 4, 3)
    # row 5 (chunk 4..7), head 3 -> kv head 1, by hand
    s = np.array([q[5, 3] @ k[j, 1] * 0.7 for j in (4, 5)])
    p = np.exp(s) / (1.0 + np.exp(s).sum())
    assert np.allclose(out[5, 3], p[0] * v[4, 1] + p[1] * v[5, 1])
    # the first row of a chunk sees itself only
    s8 = q[8, 0] @ k[8, 0] * 0.7
    assert np.allclose(out[8, 0], np.exp(s8) / (1 + np.exp(s8)) * v[8, 0])


def test_clamped_glu_by_hand():
    h = np.array([[1.0, -2.0]])
    wg, wu, wd = np.array([[3.0, 0.0], [0.0, 1.0]]), np.array([[0.0, 2.0], [1.0, 0.0]]), np.eye(2)
    # g = min((3, -2), 1.5) = (1.5, -2); u = clamp((-4, 1), +-1.5) = (-1.5, 1)
    g = np.array([1.5, -2.0])
    want = g / (1 + np.exp(-1.702 * g)) * (np.array([-1.5, 1.0]) + 1.0)
    assert np.allclose(R.clamped_glu(h, wg, wu, wd, 1.5), [want])


def test_streams_read_and_write():
    xs = np.arange(12.0).reshape(2, 2, 3)                           # [streams, rows, width]
    assert np.allclose(R.hyper_read(xs, np.array([2.0, -1.0])), 2 * xs[0] - xs[1])
    y = np.ones((2, 3))
    mix = np.array([[1.0, 2.0], [3.0, 4.0]])                        # [from, to]
    new = R.hyper_write(xs, y, mix, np.array([10.0, 20.0]))
    assert np.allclose(new[0], xs[0] + 3 * xs[1] + 10) and np.allclose(new[1], 2 * xs[0] + 4 * xs[1] + 20)


@pytest.mark.parametrize("name", ["RA", "RB", "RD"])
def test_plain_prefill_equals_plain_decoding(name):
    cfg, w = oracle(model_folder(name))
    toks = tokens_for(name, 30, 5)
    whole = R.forward(cfg, w, toks)
    mem = R.Memory()
    parts = [R.forward(cfg, w, toks[:11], mem), R.forward(cfg, w, toks[11:13], mem)]
    parts += [R.forward(cfg, w, [t], mem) for t in toks[13:]]
    assert np.allclose(np.concatenate(parts), whole, atol=1e-9)


# ------------------------------------------------------------------------------------------- configuration and parts
def test_config_is_read_whole():
    _, cfg, spec = describe_model(TINY_RA)
    assert (cfg.vocab, cfg.width, cfg.streams, cfg.eps, cfg.logit_scale) == (97, 48, 3, 1e-5, 0.75)
    m0, m1, m2, m3 = (l.mixer for l in cfg.layers)
    assert (m0.heads, m0.kv_heads, m0.dim, m0.vdim, m0.conv, m0.chunk, m0.kv_from) == (4, 2, 24, 16, 3, 7, None)
    assert m1.kv_from == 0 and cfg.layers[1].mlp is None and m2.chunk is None and m3.chunk == 20
    assert cfg.layers[3].mlp.limit == 0.5 and cfg.layers[0].mlp.ff == 80
    assert [e.cache_of for e in spec.plan] == [None, 0, None, 2] and spec.streams == 3
    _, cfg, spec = describe_model(TINY_RD)
    assert cfg.streams == 1 and not cfg.has_stream_weights and cfg.layers[0].mixer.conv == 1
    ps = DecoderModel(spec).param_specs()
    assert ps["l0.mix.q.conv"].shape == (32, 1) and DecoderModel(spec).cache_needs()[0] == PagedKeysValues(2, 16, 16)


@pytest.mark.parametrize("change, word", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].__setitem__("type", "recurrent"), "recurrent"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("heads", 3), "multiple"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_from", 1), "earlier"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 1), "no keys of its own"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("vdim", 8), "equal those"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "experts"), "experts"),
    (lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("size", 0), "size"),
])
def test_config_errors_name_the_key(change, word):
    c = copy.deepcopy(TINY_RA)
    change(c)
    with pytest.raises(ConfigError, match=word):
        describe_model(c)


def test_tensor_names_and_shapes():
    _, _, spec = describe_model(TINY_RA)
    ps = DecoderModel(spec).param_specs()
    assert ps["embed"].shape == (97, 48) and ps["embed.norm"].shape == (48,) and ps["head"].shape == (97, 48)
    assert ps["l0.mix.q"].shape == (96, 48) and ps["l0.mix.k"].shape == (48, 48) and ps["l0.mix.v"].shape == (32, 48)
    assert ps["l0.mix.q.b"].shape == (96,) and ps["l0.mix.v.conv"].shape == (32, 3) and ps["l0.mix.o"].shape == (48, 64)
    assert ps["l0.hc2.mix"].shape == (3, 3) and ps["l0.hc1.in"].shape == (3,) and ps["final.norm"].shape == (48,)
    # a layer that borrows keys has a q of its own and nothing of k and v; one without feed-forward has no second half
    l1 = sorted(n for n in ps if n.startswith("l1."))
    assert l1 == ["l1.hc1.in", "l1.hc1.mix", "l1.hc1.out", "l1.mix.o", "l1.mix.q", "l1.mix.q.b", "l1.mix.q.conv",
                  "l1.norm1"]
    _, _, spec = describe_model(TINY_RB)
    assert "l0.mix.q.conv" not in DecoderModel(spec).param_specs()       # no convolution, no taps


def test_weights_without_stream_tensors_load_and_extra_ones_are_refused():
    from allpaca_amd.weights.loader import WeightsError, load_tensors
    folder = model_folder("RD")
    _, _, spec = describe_model(TINY_RD)
    wanted = DecoderModel(spec).param_specs()
    got = load_tensors(folder, wanted, torch.float32)
    assert "l0.hc1.in" not in got and "l0.mix.q" in got
    _, _, spec = describe_model(TINY_RA)
    with pytest.raises(WeightsError):
        load_tensors(folder, DecoderModel(spec).param_specs(), torch.float32)


def test_cache_needs_and_views_of_owners_and_borrowers():
    from allpaca_amd.cache import CacheManager
    from allpaca_amd.parts import FixedState, PagedKeysValues
    _, _, spec = describe_model(TINY_RA)
    model = DecoderModel(spec)
    needs = model.cache_needs()
    assert needs[0] == {"mixer": PagedKeysValues(2, 24, 16), "mixer.state": FixedState((2, 96 + 48 + 32))}
    assert needs[1] == {"mixer.state": FixedState((2, 96))}             # its own q rows, another entry's pages
    assert needs[2]["mixer"] == PagedKeysValues(4, 16, 16) and needs[2]["mixer.state"] == FixedState((1, 64 + 64 + 64))
    assert needs[3] == {"mixer.state": FixedState((3, 64))}
    cm = CacheManager(needs, 4, 8, 2)
    assert len(cm.paged_groups) == 2 and len(cm.state_groups) == 4
    assert PagedKeysValues(2, 24, 16).page_shape(4) == (2, 4 * 40)
    _, _, spec = describe_model(TINY_RB)
    needs = DecoderModel(spec).cache_needs()
    assert needs[0] == PagedKeysValues(1, 40, 12)                       # no convolution: pages only
