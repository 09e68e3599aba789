"""The Nodupel configuration on the CPU: what the reader takes from config.json and from the weights' shapes, the run
order with its passes, the descriptions it builds, the tensors it expects, and what it refuses."""
import copy

import numpy as np
import pytest

import gpullama3_java_amd as g
import plain_nodupel as P
from gpullama3_java_amd.config import ConfigError, load_config
from gpullama3_java_amd.config.specs import Remix
from gpullama3_java_amd.parts.model import DecoderModel, expected_tensors
from nodupel_models import CONFIGS, RANKS, model


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_expected_tensors_are_the_folders_and_the_dictionary_comes_back(name):
    folder, cfg, W = model(name)
    c = load_config(folder)
    assert c.architecture == "Nodupel" and c.vocab_size == cfg["vocab"] and c.width == cfg["width"]
    exp = expected_tensors(c.model_spec())
    assert {k: tuple(v.shape) for k, v in exp.items()} == {k: tuple(v.shape) for k, v in W.items()}
    again = g.config_from_dict(c.to_dict())
    assert again == c
    # the decay's inner size is the weights': without them the reader cannot know it
    ranks = [r for r in c.decay_rank if r]
    assert ranks and all(r == RANKS[name] for r in ranks)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_run_order_and_the_mixture_in_front_of_every_pass(name):
    cfg = CONFIGS[name]
    c = g.config_from_dict(cfg)
    runs = c.run_order()
    plain = P.Sequence.run_order(cfg)
    assert [r.layer for r in runs] == [i for i, _ in plain]
    assert [isinstance(r.before, Remix) for r in runs] == [s for _, s in plain]
    spec = c.model_spec()
    assert ("loop.in" in expected_tensors(spec)) == bool(cfg.get("loop"))


def test_descriptions_carry_every_size_and_constant():
    cfg = CONFIGS["looped"]
    spec = g.config_from_dict(cfg).model_spec()
    assert spec.embedding_scale == 9.5 and spec.logit_softcap == 20.0
    pair = spec.pair_embedding
    assert (pair.buckets, pair.mul_prev, pair.mul_cur) == (211, 7, 13)
    side = spec.layers[0].mixer
    assert side.kind == "side_by_side" and side.weight == 0.5 and side.out_mult == 0.7
    left, right = side.left, side.right
    assert (left.n_heads, left.n_kv_heads, left.head_dim, left.v_head_dim) == (4, 2, 32, 48)
    assert (left.window, left.keep_first, left.scale) == (37, 5, 0.2)
    assert left.position.head_dim == 16 and left.position.scaling.factor == 4.0 and left.position.theta == 10000.0
    assert left.value_position.head_dim == 48 and left.value_position.scaling is None
    assert (right.n_heads, right.head_dim) == (3, 24)
    assert spec.layers[1].mixer.kind == "mingru" and spec.layers[1].mixer.width == 72 and spec.layers[1].mixer.out_mult == 0.7
    assert spec.layers[0].ffn.activation == "gelu_tanh" and spec.layers[0].ffn.out_mult == 0.7
    assert spec.layers[2].ffn is None and spec.layers[2].ffn_norm is None
    # a straight model: no soft cap, the whole causal range
    s2 = g.config_from_dict(CONFIGS["straight"]).model_spec()
    assert s2.logit_softcap is None and s2.layers[1].mixer.left.window is None and s2.layers[1].mixer.left.keep_first == 0


def test_cache_and_state_needs():
    import torch
    c = g.config_from_dict(CONFIGS["loop_at_end"])
    m = DecoderModel(c.model_spec(), torch.float32, "cpu")
    kv, state = m.cache_needs()
    assert len(kv) == len(state) == len(c.run_order()) + 1          # the last one holds every sequence's previous token
    assert state[-1].elements == 1 and state[-1].dtype == torch.int32
    assert kv[0].keep_first == 70 and kv[0].window == 9 and kv[1] is None
    assert state[1].elements == 50                                     # the minGRU's channels
    assert state[0].elements >= 64 + 2 * 32 * 32                       # the held row and two heads' matrices


def test_linear_scaling_divides_every_frequency():
    from gpullama3_java_amd.config.specs import LinearRopeScaling
    from gpullama3_java_amd.parts.rotary import frequencies
    plain = frequencies(16, 10000.0, None)
    scaled = frequencies(16, 10000.0, LinearRopeScaling(4.0))
    np.testing.assert_allclose(scaled, plain / 4.0, rtol=1e-7)
    np.testing.assert_allclose(plain, [10000.0 ** (-2.0 * i / 16) for i in range(8)], rtol=1e-6)


@pytest.mark.parametrize("change, word", [
    (lambda d: d["layers"][0].update(type="conv"), "type"),
    (lambda d: d["layers"][0]["mixer"]["left"].update(heads=3), "multiple"),
    (lambda d: d["layers"][0]["mixer"]["left"]["rot"].update(dims=34), "rotated"),
    (lambda d: d["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "rotated"),
    (lambda d: d["loop"].update(stop=9), "loop"),
    (lambda d: d["embedding"]["bigram"].update(buckets=0), "buckets"),
    (lambda d: d.pop("residual_mult"), "residual_mult"),
    (lambda d: d["layers"][1]["mlp"].update(kind="experts"), "mlp"),
])
def test_what_the_reader_refuses(change, word):
    d = copy.deepcopy(CONFIGS["looped"])
    change(d)
    with pytest.raises(ConfigError, match=word):
        g.config_from_dict(d)


def test_pages_of_kept_keys_stay_with_the_sequence():
    """A window gives pages back as it moves on, but never those of the first keys that stay visible."""
    import torch
    from gpullama3_java_amd.cache.kv_cache import KVNeed
    from gpullama3_java_amd.cache.pages import PagePool, SlotTable

    class Bookkeeping:                    # the cache's bookkeeping without its device memory
        pass
    from gpullama3_java_amd.cache import kv_cache
    c = Bookkeeping()
    c.page_size, c.max_pages_per_seq = 32, 64
    need = KVNeed(1, 16, window=20, keep_first=40)
    grp = Bookkeeping()
    grp.need, grp.pool, grp.dirty = need, PagePool(80), {}
    grp.table_host = np.zeros((3, 64), np.int32)
    c.groups, c.slots = [grp], SlotTable(2, 1)
    s = c.slots.take()
    c.slots.pages[s][0] = grp.pool.take(10)
    held = list(c.slots.pages[s][0])
    c._table_set = lambda g_, slot, first, pages: kv_cache.Cache._table_set(c, g_, slot, first, pages)
    kv_cache.Cache.advance(c, s, 300)
    pages = c.slots.pages[s][0]
    assert pages[:2] == held[:2]                       # positions 0 .. 39 lie in the first two pages
    assert pages[2:8] == [0] * 6                       # out of the window: given back
    assert pages[8:] == held[8:]                       # position 300 reads from 281 on: page 8
